// libmlpsp_hip: tile-centre-order forward render, scalar f32 (the bit-exact path).
//
// One 64-lane wavefront owns 64 pixels of one tile (an 8x8 tile is one wavefront; a 16x16 tile is
// four independent wavefronts, which is equivalent to the reference's block-wide exit test because
// a pixel below the transmittance floor never blends again).  The wavefront walks the tile's
// primitives in sorted order.  Per primitive:
//   * the 64-byte geometry record and the whole MLP weight block are wave-uniform, so they are
//     fetched with scalar loads into SGPRs and feed v_fma_f32 directly -- no LDS staging, no
//     barriers, no per-lane weight traffic;
//   * every live lane runs the hit test; if no lane hits, the weight block is never touched;
//   * hitting lanes evaluate the MLP in the reference's accumulation order and blend.
// The walk ends when no lane has transmittance >= 1e-3.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"

namespace mlpsp {

template <int HT, int FT>
__global__ __launch_bounds__(64) void render_tilecenter_f32_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, MlpPtrs mlp, int N, int H, TileGeom g, int waves_per_tile, int per_xcd,
    int num_items, float thr, float* __restrict__ out_rgb, float* __restrict__ out_alpha, float* __restrict__ out_t,
    unsigned long long* __restrict__ counters) {
  // XCD-aware work assignment: XCD k (blockIdx.x % 8) walks items [k*per_xcd, (k+1)*per_xcd).
  const int item = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (item >= num_items) return;
  const int tile = item / waves_per_tile;
  const int slot = (item % waves_per_tile) * 64 + threadIdx.x;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int lx = slot % g.TW, ly = slot / g.TW;
  const int x = tx * g.TW + lx, y = ty * g.TH + ly;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;

  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f;
  const float roy = valid ? rays_o[pix * 3 + 1] : 0.f;
  const float roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f;
  const float rdy = valid ? rays_d[pix * 3 + 1] : 0.f;
  const float rdz = valid ? rays_d[pix * 3 + 2] : 0.f;

  const int start = offsets[tile];
  const int end = offsets[tile + 1];

  PixelAcc acc = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
  unsigned n_proc = 0, n_proc_hit = 0, n_hits = 0;

  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool live = valid && (acc.trans >= kTransmittanceFloor);
    const bool hit = live && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    const unsigned long long hit_mask = __ballot(hit);
    ++n_proc;
    if (hit_mask != 0ull) {
      ++n_proc_hit;
      n_hits += __popcll(hit_mask);
      if (hit) {
        const float x6[6] = {rdx, rdy, rdz, h.dx, h.dy, h.dz};
        float o[4];
        mlp_eval<HT, FT>(x6, freq, att, F, H, mlp, p, o);
        blend_step(acc, o[0], o[1], o[2], o[3], h.decay, h.t);
      }
    }
    if (__ballot(valid && (acc.trans >= kTransmittanceFloor)) == 0ull) break;
  }

  if (valid) {
    out_rgb[pix * 3 + 0] = acc.cr;
    out_rgb[pix * 3 + 1] = acc.cg;
    out_rgb[pix * 3 + 2] = acc.cb;
    out_alpha[pix] = 1.f - acc.trans;
    if (out_t) out_t[pix] = acc.t_acc / (acc.w_acc > 1e-8f ? acc.w_acc : 1.f);
  }
  if (counters && threadIdx.x == 0) {
    atomicAdd(counters + 1, (unsigned long long)n_proc);
    atomicAdd(counters + 2, (unsigned long long)n_proc_hit);
    atomicAdd(counters + 3, (unsigned long long)n_hits);
  }
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_render_tilecenter_f32(const float* rays_o_dev, const float* rays_d_dev,
                                          const void* prim_records_dev, const int32_t* order_dev,
                                          const int32_t* tile_offsets_dev, const float* freq_dev,
                                          const float* att_dev, int num_frequencies, const float* W1,
                                          const float* b1, const float* W2, const float* b2, const float* W3,
                                          const float* b3, int num_primitives, int hidden, int width, int height,
                                          int tile_w, int tile_h, float threshold, float* out_rgb_dev,
                                          float* out_alpha_dev, float* out_t_dev, int64_t* counters_dev,
                                          mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 64 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !out_rgb_dev || !out_alpha_dev) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  const int per_xcd = (int)((items + kNumXcd - 1) / kNumXcd);
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  MlpPtrs m{W1, b1, W2, b2, W3, b3};
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
  hipStream_t s = (hipStream_t)stream;
  auto* ctr = reinterpret_cast<unsigned long long*>(counters_dev);
#define MLPSP_F32_LAUNCH(HT, FT)                                                                                  \
  hipLaunchKernelGGL((render_tilecenter_f32_kernel<HT, FT>), grid, block, 0, s, rays_o_dev, rays_d_dev,           \
                     (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,         \
                     num_frequencies, m, num_primitives, hidden, g, wpt, per_xcd, (int)items, threshold,           \
                     out_rgb_dev, out_alpha_dev, out_t_dev, ctr)
  if (hidden == 32 && num_frequencies == 6) MLPSP_F32_LAUNCH(32, 6);
  else if (hidden == 16 && num_frequencies == 6) MLPSP_F32_LAUNCH(16, 6);
  else MLPSP_F32_LAUNCH(0, 0);
#undef MLPSP_F32_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
