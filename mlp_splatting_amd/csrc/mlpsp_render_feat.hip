// libmlpsp_hip: tile-centre-order forward with the gated per-primitive feature channel, scalar f32.
//
// The reference read-modify-writes a C-float row of global memory per hit and per pixel
// (np_tile_kernels.cu:6036-6075).  Here the work is split in two kernels that keep the reference's
// arithmetic order per pixel and channel (feat = fma(w, mix, feat), mix the fma chain over the slots),
// so the result is bit-identical to a sequential evaluation:
//   1. the f32 render kernel (lane = pixel, mlpsp_render_f32.hpp) composites RGB and emits, per wavefront,
//      the primitives that hit and per pixel the weight w and the four gates (hit records,
//      mlpsp_hitrec.hpp): float[K][64] with K = 5 (w, g0..g3) or 1 (w), w = -1 where the primitive missed;
//   2. feat_accumulate_kernel turns the roles around: lane = channel.  A 256-thread block owns one
//      64-pixel item; wavefront v owns channels [128v, 128v+128) of all 64 pixels in 128 accumulator
//      VGPRs.  Per record the attribute rows are two coalesced loads per slot, the per-pixel weight and
//      gates are wave-uniform scalar operands, a pixel the primitive missed costs one scalar branch, and
//      every output row is written exactly once.
#include "mlpsp_device.hpp"
#include "mlpsp_hitrec.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"
#include "mlpsp_render_f32.hpp"

namespace mlpsp {

typedef float f32x8 __attribute__((ext_vector_type(8)));

// SLOTS = 1, 4 or 5; mix as np_tile_kernels.cu:6037-6070.
template <int SLOTS>
__global__ __launch_bounds__(256) void feat_accumulate_kernel(const float* __restrict__ feat_attr, int C, HitPool hp,
                                                              const int32_t* __restrict__ offsets, TileGeom g,
                                                              int waves_per_tile, int per_xcd, int num_items,
                                                              float* __restrict__ out_feat) {
  const int item = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (item >= num_items) return;
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const int c0 = ((int)blockIdx.y * 4 + wave) * 128;
  if (c0 >= C) return;
  const int tile = item / waves_per_tile, wslot = item % waves_per_tile;
  const int hits = hp.item_hits[item];
  const int table_base = wslot * hp.table_stride + (offsets[tile] >> 4) + tile;
  const int ca = c0 + l, cb = c0 + 64 + l;
  const bool has_a = ca < C, has_b = cb < C;
  constexpr bool GATED = SLOTS > 1;
  constexpr int K = GATED ? 5 : 1;

  float acc[64][2];
#pragma unroll
  for (int px = 0; px < 64; ++px) acc[px][0] = acc[px][1] = 0.f;

  for (int m = 0; m < hits; ++m) {
    const int rs = __builtin_amdgcn_readfirstlane(hit_slot(hp, table_base, m));
    const int p = __builtin_amdgcn_readfirstlane(hp.hit_ids[rs]);
    const float* __restrict__ rows = feat_attr + (size_t)p * SLOTS * C;
    float ra[SLOTS], rb[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      ra[s] = has_a ? rows[(size_t)s * C + ca] : 0.f;
      rb[s] = has_b ? rows[(size_t)s * C + cb] : 0.f;
    }
    const float* __restrict__ rec = reinterpret_cast<const float*>(hp.records + (size_t)rs * hp.record_bytes);
    // weights and gates of 8 pixels at a time: wave-uniform 32-byte scalar loads, issued unconditionally
    // so that their latency overlaps the previous group's arithmetic
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const f32x8 w8 = *reinterpret_cast<const f32x8*>(rec + 8 * q);
      f32x8 g8[4];
      if constexpr (GATED) {
#pragma unroll
        for (int k = 0; k < 4; ++k) g8[k] = *reinterpret_cast<const f32x8*>(rec + 64 * (k + 1) + 8 * q);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int px = 8 * q + j;
        const float w = w8[j];
        if (w >= 0.f) {
          float ma, mb;
          if constexpr (SLOTS == 1) {
            ma = ra[0];
            mb = rb[0];
          } else {
            const float g0 = g8[0][j], g1 = g8[1][j], g2 = g8[2][j], g3 = g8[3][j];
            if constexpr (SLOTS == 4) {
              ma = fmaf(g0, ra[0], 0.f);
              mb = fmaf(g0, rb[0], 0.f);
              ma = fmaf(g1, ra[1], ma);
              mb = fmaf(g1, rb[1], mb);
              ma = fmaf(g2, ra[2], ma);
              mb = fmaf(g2, rb[2], mb);
              ma = fmaf(g3, ra[3], ma);
              mb = fmaf(g3, rb[3], mb);
            } else {
              ma = fmaf(g0, ra[1], ra[0]);
              mb = fmaf(g0, rb[1], rb[0]);
              ma = fmaf(g1, ra[2], ma);
              mb = fmaf(g1, rb[2], mb);
              ma = fmaf(g2, ra[3], ma);
              mb = fmaf(g2, rb[3], mb);
              ma = fmaf(g3, ra[4], ma);
              mb = fmaf(g3, rb[4], mb);
            }
          }
          acc[px][0] = fmaf(w, ma, acc[px][0]);
          acc[px][1] = fmaf(w, mb, acc[px][1]);
        }
      }
    }
  }

  const int tx = tile % g.ntx, ty = tile / g.ntx;
#pragma unroll
  for (int px = 0; px < 64; ++px) {
    const int slot = wslot * 64 + px;
    const int x = tx * g.TW + slot % g.TW, y = ty * g.TH + slot / g.TW;
    if (slot < g.TW * g.TH && x < g.W && y < g.H) {
      float* __restrict__ dst = out_feat + (size_t)(y * g.W + x) * C;
      if (has_a) dst[ca] = acc[px][0];
      if (has_b) dst[cb] = acc[px][1];
    }
  }
  (void)K;
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_feat_workspace_bytes(int64_t num_pairs, int width, int height, int tile_w, int tile_h,
                                            int feat_slots, int fp16_records, int64_t pool_records) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (T <= 0 || tile_px <= 0 || tile_px > 256 || num_pairs < 0 || !(feat_slots == 1 || feat_slots == 4 || feat_slots == 5))
    return 0;
  const int wpt = (int)((tile_px + 63) / 64);
  const int rec = fp16_records ? 64 * 2 * (feat_slots == 5 ? 8 : 4) : 64 * 4 * (feat_slots > 1 ? 5 : 1);
  // every wavefront draws records 64 at a time: its last draw can stay 63 short of full
  const int64_t worst = num_pairs * wpt + (int64_t)(kHitChunk * kHitGrab - 1) * T * wpt + kHitChunk * kHitGrab;
  if (pool_records < 0 || pool_records > worst) pool_records = worst;
  return hitpool_bytes(num_pairs, T, wpt, pool_records, rec);
}

MLPSP_API int mlpsp_render_tilecenter_feat_f32(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* order_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, const float* feat_attr_dev, int feat_slots, int feat_channels, float gating_beta,
    float gating_temp, int width, int height, int tile_w, int tile_h, float threshold, int64_t num_pairs,
    void* workspace_dev, size_t workspace_bytes, float* out_rgb_dev, float* out_alpha_dev, float* out_feat_dev,
    int32_t* status_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 64 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (!(feat_slots == 1 || feat_slots == 4 || feat_slots == 5) || feat_channels <= 0 || feat_channels > 512)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !out_rgb_dev || !out_alpha_dev || !out_feat_dev ||
      !status_dev || num_pairs < 0 || num_pairs > 2147483647LL)
    return MLPSP_E_ARGUMENT;
  if (num_primitives > 0 && !feat_attr_dev) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  if (!workspace_dev || reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0 ||
      workspace_bytes < hitpool_min_bytes(num_pairs, T, wpt))
    return MLPSP_E_SCRATCH;
  const int rec_bytes = 64 * 4 * (feat_slots > 1 ? 5 : 1);
  const HitPool hp = hitpool_carve(workspace_dev, workspace_bytes, num_pairs, T, wpt, rec_bytes);
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(hp.counters, 0, 64 * sizeof(int32_t), s));
  const int per_xcd = (int)((items + kNumXcd - 1) / kNumXcd);
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
#define MLPSP_EMIT_LAUNCH(HT, FT, EM, ...)                                                                        \
  hipLaunchKernelGGL((render_tilecenter_f32_kernel<HT, FT, EM, ##__VA_ARGS__>), grid, block, 0, s, rays_o_dev, rays_d_dev,       \
                     (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,         \
                     num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives, hidden, g, wpt, per_xcd, (int)items, threshold,          \
                     out_rgb_dev, out_alpha_dev, (float*)nullptr, (unsigned long long*)nullptr, gating_beta,      \
                     gating_temp, hp)
  const bool gated = feat_slots > 1;
  if (hidden == 32 && use_mfma32(hidden, num_frequencies, W1, b1, W2, b2)) {
    if (gated) MLPSP_EMIT_LAUNCH(32, 6, 2, false, true);
    else MLPSP_EMIT_LAUNCH(32, 6, 1, false, true);
  } else if (hidden == 32 && num_frequencies == 6) {
    if (gated) MLPSP_EMIT_LAUNCH(32, 6, 2);
    else MLPSP_EMIT_LAUNCH(32, 6, 1);
  } else {
    if (gated) MLPSP_EMIT_LAUNCH(0, 0, 2);
    else MLPSP_EMIT_LAUNCH(0, 0, 1);
  }
#undef MLPSP_EMIT_LAUNCH
  MLPSP_LAUNCH_CHECK();
  const dim3 agrid((unsigned)(per_xcd * kNumXcd), (unsigned)ceil_div(feat_channels, 512)), ablock(256);
#define MLPSP_ACC_LAUNCH(SL)                                                                                     \
  hipLaunchKernelGGL((feat_accumulate_kernel<SL>), agrid, ablock, 0, s, feat_attr_dev, feat_channels, hp,        \
                     tile_offsets_dev, g, wpt, per_xcd, (int)items, out_feat_dev)
  if (feat_slots == 4) MLPSP_ACC_LAUNCH(4);
  else if (feat_slots == 5) MLPSP_ACC_LAUNCH(5);
  else MLPSP_ACC_LAUNCH(1);
#undef MLPSP_ACC_LAUNCH
  MLPSP_LAUNCH_CHECK();
  // status_dev[0] = 1 if the record pool was too small (the feature image is then incomplete)
  MLPSP_HIP_TRY(hipMemcpyAsync(status_dev, hp.counters + 1, sizeof(int32_t), hipMemcpyDeviceToDevice, s));
  return MLPSP_OK;
}
