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
#include "mlpsp_hitrec.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"
#include "mlpsp_render_f32.hpp"

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
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
  hipStream_t s = (hipStream_t)stream;
  auto* ctr = reinterpret_cast<unsigned long long*>(counters_dev);
#define MLPSP_F32_LAUNCH(HT, FT, ...)                                                                             \
  hipLaunchKernelGGL((render_tilecenter_f32_kernel<HT, FT, 0, ##__VA_ARGS__>), grid, block, 0, s, rays_o_dev, rays_d_dev,        \
                     (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,         \
                     num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives, hidden, g, wpt, per_xcd, (int)items, threshold,           \
                     out_rgb_dev, out_alpha_dev, out_t_dev, ctr, 0.f, 0.f, HitPool{})
#define MLPSP_F32_AHEAD_LAUNCH(HT, HALF, UNITS)                                                                   \
  hipLaunchKernelGGL((render_tilecenter_f32_ahead_kernel<HT, HALF>), dim3((unsigned)(ceil_div_units(UNITS) * kNumXcd)), block, 0, s, \
                     rays_o_dev, rays_d_dev, (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev,    \
                     freq_dev, att_dev, W1, b1, W2, b2, W3, b3, num_primitives, g, wpt, ceil_div_units(UNITS),    \
                     (int)(UNITS), threshold, out_rgb_dev, out_alpha_dev, out_t_dev, ctr)
  const auto ceil_div_units = [](int64_t units) { return (int)((units + kNumXcd - 1) / kNumXcd); };
  if (use_mfma32(hidden, num_frequencies, W1, b1, W2, b2)) {
    const int mode = ahead_mode(items, num_primitives, ctr != nullptr);
    if (mode == 2) {
      if (hidden == 32) MLPSP_F32_AHEAD_LAUNCH(32, true, 2 * items);
      else MLPSP_F32_AHEAD_LAUNCH(16, true, 2 * items);
    } else if (mode == 1) {
      if (hidden == 32) MLPSP_F32_AHEAD_LAUNCH(32, false, items);
      else MLPSP_F32_AHEAD_LAUNCH(16, false, items);
    } else if (hidden == 32) MLPSP_F32_LAUNCH(32, 6, false, true);
    else MLPSP_F32_LAUNCH(16, 6, false, true);
  }
  else if (hidden == 32 && num_frequencies == 6) MLPSP_F32_LAUNCH(32, 6);
  else if (hidden == 16 && num_frequencies == 6) MLPSP_F32_LAUNCH(16, 6);
  else MLPSP_F32_LAUNCH(0, 0);
#undef MLPSP_F32_AHEAD_LAUNCH
#undef MLPSP_F32_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_render_tilecenter_stats_f32(const float* rays_o_dev, const float* rays_d_dev,
                                                const void* prim_records_dev, const int32_t* order_dev,
                                                const int32_t* tile_offsets_dev, const float* freq_dev,
                                                const float* att_dev, int num_frequencies, const float* W1,
                                                const float* b1, const float* W2, const float* b2, const float* W3,
                                                const float* b3, int num_primitives, int hidden, int width,
                                                int height, int tile_w, int tile_h, float threshold,
                                                const float* gt_rgb_dev, float* out_rgb_dev, float* out_alpha_dev,
                                                float* stat_sum_w_dev, float* stat_max_w_dev, int32_t* stat_hits_dev,
                                                float* stat_sum_werr_dev, int32_t* stat_contrib_dev,
                                                mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 64 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !out_rgb_dev || !out_alpha_dev || !gt_rgb_dev)
    return MLPSP_E_ARGUMENT;
  if (num_primitives > 0 && (!stat_sum_w_dev || !stat_max_w_dev || !stat_hits_dev)) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  const int per_xcd = (int)((items + kNumXcd - 1) / kNumXcd);
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
  hipStream_t s = (hipStream_t)stream;
#define MLPSP_STATS_LAUNCH(HT, FT, ...)                                                                          \
  hipLaunchKernelGGL((render_tilecenter_f32_kernel<HT, FT, 0, true, ##__VA_ARGS__>), grid, block, 0, s, rays_o_dev, rays_d_dev, \
                     (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,        \
                     num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives, hidden, g, wpt, per_xcd,           \
                     (int)items, threshold, out_rgb_dev, out_alpha_dev, (float*)nullptr,                         \
                     (unsigned long long*)nullptr, 0.f, 0.f, HitPool{}, gt_rgb_dev, stat_sum_w_dev,              \
                     stat_max_w_dev, stat_hits_dev, stat_sum_werr_dev, stat_contrib_dev)
  if (use_mfma32(hidden, num_frequencies, W1, b1, W2, b2)) {
    if (hidden == 32) MLPSP_STATS_LAUNCH(32, 6, true);
    else MLPSP_STATS_LAUNCH(16, 6, true);
  }
  else if (hidden == 32 && num_frequencies == 6) MLPSP_STATS_LAUNCH(32, 6);
  else if (hidden == 16 && num_frequencies == 6) MLPSP_STATS_LAUNCH(16, 6);
  else MLPSP_STATS_LAUNCH(0, 0);
#undef MLPSP_STATS_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
