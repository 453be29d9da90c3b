// libmlpsp_hip: tile-centre-order forward with the gated per-primitive feature channel, scalar f32.
//
// The reference read-modify-writes a C-float row of global memory per hit and per pixel
// (np_tile_kernels.cu:6036-6075).  Here a wavefront keeps lane = pixel and owns a chunk of 128
// channels in 128 accumulator VGPRs; the primitive's feature rows are wave-uniform and arrive as
// scalar operands, so one hit costs 5 v_fma per channel and no memory traffic but the attribute
// rows themselves.  grid.y walks the channel chunks (each chunk repeats the cheap traversal);
// every output row is written exactly once, as 16-byte stores.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_feat.hpp"
#include "mlpsp_mlp.hpp"

namespace mlpsp {

template <int HT, int FT, int SLOTS>
__global__ __launch_bounds__(64) void render_tilecenter_feat_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, MlpPtrs mlp, const float* __restrict__ feat_attr, int C, float beta,
    float temp, int N, int H, TileGeom g, int waves_per_tile, int per_xcd, int num_items, float thr,
    float* __restrict__ out_rgb, float* __restrict__ out_alpha, float* __restrict__ out_feat) {
  const int item = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (item >= num_items) return;
  const int c0 = blockIdx.y * kFeatChunk;
  const int nch = min(kFeatChunk, C - c0);
  const int tile = item / waves_per_tile;
  const int slot = (item % waves_per_tile) * 64 + threadIdx.x;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int x = tx * g.TW + slot % g.TW, y = ty * g.TH + slot / g.TW;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f, roy = valid ? rays_o[pix * 3 + 1] : 0.f,
              roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f, rdy = valid ? rays_d[pix * 3 + 1] : 0.f,
              rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  const int start = offsets[tile], end = offsets[tile + 1];

  PixelAcc pa = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
  float acc[kFeatChunk];
#pragma unroll
  for (int j = 0; j < kFeatChunk; ++j) acc[j] = 0.f;

  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool live = valid && (pa.trans >= kTransmittanceFloor);
    const bool hit = live && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    if (__ballot(hit) != 0ull) {
      if (hit) {
        const float x6[6] = {rdx, rdy, rdz, h.dx, h.dy, h.dz};
        float o[4];
        mlp_eval<HT, FT>(x6, freq, att, F, H, mlp, p, o);
        const float w = blend_step(pa, o[0], o[1], o[2], o[3], h.decay, h.t);
        float gt[4] = {0.f, 0.f, 0.f, 0.f};
        if constexpr (SLOTS > 1) tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
        const float* __restrict__ rows = feat_attr + (size_t)p * SLOTS * C + c0;
        feat_chunk_accumulate<SLOTS>(acc, rows, C, nch, w, gt);
      }
    }
    if (__ballot(valid && (pa.trans >= kTransmittanceFloor)) == 0ull) break;
  }

  if (valid) {
    if (blockIdx.y == 0) {
      out_rgb[pix * 3 + 0] = pa.cr;
      out_rgb[pix * 3 + 1] = pa.cg;
      out_rgb[pix * 3 + 2] = pa.cb;
      out_alpha[pix] = 1.f - pa.trans;
    }
    feat_chunk_store(acc, out_feat + (size_t)pix * C + c0, C, nch);
  }
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_render_tilecenter_feat_f32(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* order_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, const float* feat_attr_dev, int feat_slots, int feat_channels, float gating_beta,
    float gating_temp, int width, int height, int tile_w, int tile_h, float threshold, float* out_rgb_dev,
    float* out_alpha_dev, float* out_feat_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 64 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (!(feat_slots == 1 || feat_slots == 4 || feat_slots == 5) || feat_channels <= 0 || feat_channels > 512)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !out_rgb_dev || !out_alpha_dev || !out_feat_dev)
    return MLPSP_E_ARGUMENT;
  if (num_primitives > 0 && !feat_attr_dev) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  const int per_xcd = (int)((items + kNumXcd - 1) / kNumXcd);
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  MlpPtrs m{W1, b1, W2, b2, W3, b3};
  const dim3 grid((unsigned)(per_xcd * kNumXcd), (unsigned)ceil_div(feat_channels, kFeatChunk)), block(64);
  hipStream_t s = (hipStream_t)stream;
#define MLPSP_FEAT_LAUNCH(HT, FT, SL)                                                                              \
  hipLaunchKernelGGL((render_tilecenter_feat_kernel<HT, FT, SL>), grid, block, 0, s, rays_o_dev, rays_d_dev,       \
                     (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,          \
                     num_frequencies, m, feat_attr_dev, feat_channels, gating_beta, gating_temp, num_primitives,    \
                     hidden, g, wpt, per_xcd, (int)items, threshold, out_rgb_dev, out_alpha_dev, out_feat_dev)
#define MLPSP_FEAT_SLOTS(HT, FT)                       \
  do {                                                 \
    if (feat_slots == 4) MLPSP_FEAT_LAUNCH(HT, FT, 4); \
    else if (feat_slots == 5) MLPSP_FEAT_LAUNCH(HT, FT, 5); \
    else MLPSP_FEAT_LAUNCH(HT, FT, 1);                 \
  } while (0)
  if (hidden == 32 && num_frequencies == 6) MLPSP_FEAT_SLOTS(32, 6);
  else MLPSP_FEAT_SLOTS(0, 0);
#undef MLPSP_FEAT_SLOTS
#undef MLPSP_FEAT_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
