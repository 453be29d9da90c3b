// libmlpsp_hip: per-pixel-order forward (each pixel blends its own hits sorted by its own t), f32.
//
// Reference: render_tiles_kernel_with_sort / _and_feat (np_tile_kernels.cu:715-926, 929-1208):
// gather up to 256 hits per pixel in list order, insertion-sort them by t (strict '>', i.e. stable),
// blend until T < 1e-3.  Here lane = pixel and a wavefront owns 64 pixels of a tile:
//   gather : walk the tile list once (wave-uniform primitive, scalar geometry loads); every hitting
//            lane appends (t, list position) to its column of a [256][64] workspace block, so the
//            wavefront's appends and later reads are coalesced;
//   blend  : instead of sorting, each step selects the smallest (t, list position) pair above the
//            last one blended -- the same sequence a stable sort yields -- and stops as soon as the
//            pixel falls below the transmittance floor, which in practice is long before the list
//            is exhausted.  The hit geometry is recomputed (same operations, same bits) rather than
//            stored, which keeps the workspace at 8 bytes per hit.
// In this mode neighbouring lanes blend different primitives, so geometry and weights are
// per-lane gathers; it is the quality-reference ordering, not the fast path.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"

namespace mlpsp {

constexpr int kHitCap = MLPSP_PIXEL_HIT_CAPACITY;
constexpr int kPPChunk = 128;

template <int HT, int FT, bool FEAT>
__global__ __launch_bounds__(64) void render_per_pixel_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ cand, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, MlpPtrs mlp, const float* __restrict__ feat_attr, int slots, int C,
    float beta, float temp, int N, int H, TileGeom g, int waves_per_tile, int num_items, float thr,
    float* __restrict__ ws_t, int32_t* __restrict__ ws_k, int32_t* __restrict__ overflow,
    float* __restrict__ out_rgb, float* __restrict__ out_alpha, float* __restrict__ out_feat) {
  const int item = blockIdx.x;
  if (item >= num_items) return;
  const int lane = threadIdx.x;
  const int tile = item / waves_per_tile;
  const int slot = (item % waves_per_tile) * 64 + lane;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int x = tx * g.TW + slot % g.TW, y = ty * g.TH + slot / g.TW;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f, roy = valid ? rays_o[pix * 3 + 1] : 0.f,
              roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f, rdy = valid ? rays_d[pix * 3 + 1] : 0.f,
              rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  const int start = offsets[tile], end = offsets[tile + 1];
  float* __restrict__ my_t = ws_t + (size_t)item * kHitCap * 64 + lane;
  int32_t* __restrict__ my_k = ws_k + (size_t)item * kHitCap * 64 + lane;

  // ---- gather (np_tile_kernels.cu:775-811): the 257th hit raises the flag and ends the gather
  int cnt = 0;
  bool gathering = valid;
  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(cand[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool hit = gathering && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    if (hit) {
      if (cnt < kHitCap) {
        my_t[cnt * 64] = h.t;
        my_k[cnt * 64] = i - start;
        ++cnt;
      } else {
        atomicExch(overflow, 1);
        gathering = false;
      }
    }
    if (__ballot(gathering) == 0ull) break;
  }

  // ---- blend, one channel chunk at a time (a single pass when there is no feature output)
  constexpr int kAcc = FEAT ? kPPChunk : 1;
  const int nchunks = FEAT ? (C + kPPChunk - 1) / kPPChunk : 1;
  for (int chunk = 0; chunk < nchunks; ++chunk) {
    const int c0 = chunk * kPPChunk;
    const int nch = FEAT ? min(kPPChunk, C - c0) : 0;
    PixelAcc pa = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
    float acc[kAcc];
#pragma unroll
    for (int j = 0; j < kAcc; ++j) acc[j] = 0.f;
    float last_t = -1.f;
    int last_k = -1;
    for (int step = 0;; ++step) {
      const bool active = (step < cnt) && (pa.trans >= kTransmittanceFloor);
      if (__ballot(active) == 0ull) break;
      if (active) {
        float best_t = __builtin_inff();
        int best_k = 0x7fffffff;
        for (int s = 0; s < cnt; ++s) {
          const float t = my_t[s * 64];
          const int k = my_k[s * 64];
          const bool after = (t > last_t) || (t == last_t && k > last_k);
          const bool better = (t < best_t) || (t == best_t && k < best_k);
          if (after && better) {
            best_t = t;
            best_k = k;
          }
        }
        last_t = best_t;
        last_k = best_k;
        const int p = cand[start + best_k];
        const PrimRecord P = prims[p];
        HitInfo h;
        (void)hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
        const float x6[6] = {rdx, rdy, rdz, h.dx, h.dy, h.dz};
        float o[4];
        mlp_eval<HT, FT>(x6, freq, att, F, H, mlp, p, o);
        const float w = blend_step(pa, o[0], o[1], o[2], o[3], h.decay, h.t);
        if constexpr (FEAT) {
          float gt[4] = {0.f, 0.f, 0.f, 0.f};
          if (slots > 1) tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
          const float* __restrict__ rows = feat_attr + (size_t)p * slots * C + c0;
#pragma unroll
          for (int j = 0; j < kPPChunk; ++j) {
            if (j < nch) {
              float mix;
              if (slots <= 1) {
                mix = rows[j];
              } else if (slots == 5) {
                mix = rows[j];
                mix = fmaf(gt[0], rows[C + j], mix);
                mix = fmaf(gt[1], rows[2 * C + j], mix);
                mix = fmaf(gt[2], rows[3 * C + j], mix);
                mix = fmaf(gt[3], rows[4 * C + j], mix);
              } else {
                mix = fmaf(gt[0], rows[j], 0.f);
                mix = fmaf(gt[1], rows[C + j], mix);
                mix = fmaf(gt[2], rows[2 * C + j], mix);
                mix = fmaf(gt[3], rows[3 * C + j], mix);
              }
              acc[j] = fmaf(w, mix, acc[j]);
            }
          }
        }
      }
    }
    if (valid) {
      if (chunk == 0) {
        out_rgb[pix * 3 + 0] = pa.cr;
        out_rgb[pix * 3 + 1] = pa.cg;
        out_rgb[pix * 3 + 2] = pa.cb;
        out_alpha[pix] = 1.f - pa.trans;
      }
      if constexpr (FEAT) {
        float* __restrict__ dst = out_feat + (size_t)pix * C + c0;
#pragma unroll
        for (int j = 0; j < kPPChunk; ++j)
          if (j < nch) dst[j] = acc[j];
      }
    }
  }
}

// Training records in per-pixel order: the traversal of render_tiles_backward_count_per_pixel / _emit_per_pixel
// (np_tile_kernels.cu:1211-1836) with the record schema of the tile-centre records forward (:3138-3154) and the
// record kernels' MLP arithmetic (mlp_eval_rgb_sigma).  Same gather and select-min walk as the render kernel above;
// EMIT = false leaves the number of blended hits per pixel, EMIT = true writes record k of a pixel at
// rec_offsets[pixel] + k together with the image.  Both passes gather again: the workspace is the render's.
template <int HT, int FT, bool EMIT>
__global__ __launch_bounds__(64) void records_per_pixel_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ cand, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, MlpPtrs mlp, float beta, float temp, int N, int H, TileGeom g,
    int waves_per_tile, int num_items, float thr, float* __restrict__ ws_t, int32_t* __restrict__ ws_k,
    int32_t* __restrict__ overflow, int32_t* __restrict__ counts, const long long* __restrict__ rec_offsets,
    int32_t* __restrict__ out_ids, float* __restrict__ out_x6, int32_t* __restrict__ out_masks,
    float* __restrict__ out_raw, float* __restrict__ out_gates, float* __restrict__ out_rgb,
    float* __restrict__ out_alpha) {
  const int item = blockIdx.x;
  if (item >= num_items) return;
  const int lane = threadIdx.x;
  const int tile = item / waves_per_tile;
  const int slot = (item % waves_per_tile) * 64 + lane;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int x = tx * g.TW + slot % g.TW, y = ty * g.TH + slot / g.TW;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f, roy = valid ? rays_o[pix * 3 + 1] : 0.f,
              roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f, rdy = valid ? rays_d[pix * 3 + 1] : 0.f,
              rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  const int start = offsets[tile], end = offsets[tile + 1];
  float* __restrict__ my_t = ws_t + (size_t)item * kHitCap * 64 + lane;
  int32_t* __restrict__ my_k = ws_k + (size_t)item * kHitCap * 64 + lane;

  int cnt = 0;
  bool gathering = valid;
  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(cand[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool hit = gathering && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    if (hit) {
      if (cnt < kHitCap) {
        my_t[cnt * 64] = h.t;
        my_k[cnt * 64] = i - start;
        ++cnt;
      } else {
        atomicExch(overflow, 1);
        gathering = false;
      }
    }
    if (__ballot(gathering) == 0ull) break;
  }

  float trans = 1.f, cr = 0.f, cg = 0.f, cb = 0.f;
  float last_t = -1.f;
  int last_k = -1, used = 0;
  const long long rec_base = (EMIT && valid) ? rec_offsets[pix] : 0;
  for (int step = 0;; ++step) {
    const bool active = (step < cnt) && (trans >= kTransmittanceFloor);
    if (__ballot(active) == 0ull) break;
    if (active) {
      float best_t = __builtin_inff();
      int best_k = 0x7fffffff;
      for (int s = 0; s < cnt; ++s) {
        const float t = my_t[s * 64];
        const int k = my_k[s * 64];
        const bool after = (t > last_t) || (t == last_t && k > last_k);
        const bool better = (t < best_t) || (t == best_t && k < best_k);
        if (after && better) {
          best_t = t;
          best_k = k;
        }
      }
      last_t = best_t;
      last_k = best_k;
      const int p = cand[start + best_k];
      const PrimRecord P = prims[p];
      HitInfo h;
      (void)hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
      const float x6[6] = {rdx, rdy, rdz, h.dx, h.dy, h.dz};
      float o[4];
      uint32_t mk[2];
      mlp_eval<HT, FT, true>(x6, freq, att, F, H, mlp, p, o, mk);
      const float R = sigmoid(o[0]), G = sigmoid(o[1]), Bc = sigmoid(o[2]);
      const float sigma_raw = softplus(o[3]);
      const float alpha = 1.f - det_exp(-(sigma_raw * h.decay));
      if constexpr (EMIT) {
        const long long r = rec_base + used;
        out_ids[r] = p;
#pragma unroll
        for (int c = 0; c < 6; ++c) out_x6[r * 6 + c] = x6[c];
        out_masks[r * 2] = (int32_t)mk[0];
        out_masks[r * 2 + 1] = (int32_t)mk[1];
        float* __restrict__ raw = out_raw + r * 8;
        raw[0] = R;
        raw[1] = G;
        raw[2] = Bc;
        raw[3] = sigma_raw;
        raw[4] = trans;
        raw[5] = alpha;
        raw[6] = h.decay;
        raw[7] = o[3];
        float gt[4];
        tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
#pragma unroll
        for (int k = 0; k < 4; ++k) out_gates[r * 4 + k] = gt[k];
        const float weight = trans * alpha;
        cr = fmaf(weight, R, cr);
        cg = fmaf(weight, G, cg);
        cb = fmaf(weight, Bc, cb);
      }
      trans = trans * (1.f - alpha);
      ++used;
    }
  }
  if (valid) {
    if constexpr (EMIT) {
      out_rgb[pix * 3 + 0] = cr;
      out_rgb[pix * 3 + 1] = cg;
      out_rgb[pix * 3 + 2] = cb;
      out_alpha[pix] = 1.f - trans;
    } else {
      counts[pix] = used;
    }
  }
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_per_pixel_workspace_bytes(int width, int height, int tile_w, int tile_h) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (T <= 0 || tile_px <= 0 || tile_px > 256) return 0;
  const int64_t items = T * ((tile_px + 63) / 64);
  return (size_t)items * 64 * kHitCap * (sizeof(float) + sizeof(int32_t)) + 256;
}

MLPSP_API int mlpsp_render_per_pixel_f32(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* candidates_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, const float* feat_attr_dev, int feat_slots, int feat_channels, float gating_beta,
    float gating_temp, int width, int height, int tile_w, int tile_h, float threshold, void* workspace_dev,
    size_t workspace_bytes, float* out_rgb_dev, float* out_alpha_dev, float* out_feat_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 64 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (out_feat_dev) {
    if (!(feat_slots == 1 || feat_slots == 4 || feat_slots == 5) || feat_channels <= 0 || feat_channels > 512)
      return MLPSP_E_ARGUMENT;
    if (num_primitives > 0 && !feat_attr_dev) return MLPSP_E_ARGUMENT;
  }
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !out_rgb_dev || !out_alpha_dev || !workspace_dev)
    return MLPSP_E_ARGUMENT;
  const size_t need = mlpsp_per_pixel_workspace_bytes(width, height, tile_w, tile_h);
  if (workspace_bytes < need) return MLPSP_E_SCRATCH;
  if (reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  // workspace: [flag (256 B)] [t: items*256*64 f32] [k: items*256*64 i32]
  int32_t* flag = reinterpret_cast<int32_t*>(workspace_dev);
  float* ws_t = reinterpret_cast<float*>(static_cast<char*>(workspace_dev) + 256);
  int32_t* ws_k = reinterpret_cast<int32_t*>(ws_t + (size_t)items * 64 * kHitCap);
  MLPSP_HIP_TRY(hipMemsetAsync(flag, 0, sizeof(int32_t), s));
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  MlpPtrs m{W1, b1, W2, b2, W3, b3};
  const dim3 grid((unsigned)items), block(64);
#define MLPSP_PP_LAUNCH_(HT, FT, FE)                                                                                 \
  hipLaunchKernelGGL((render_per_pixel_kernel<HT, FT, FE>), grid, block, 0, s, rays_o_dev, rays_d_dev,                 \
                     (const PrimRecord*)prim_records_dev, candidates_dev, tile_offsets_dev, freq_dev, att_dev,     \
                     num_frequencies, m, feat_attr_dev, feat_slots, feat_channels, gating_beta, gating_temp,        \
                     num_primitives, hidden, g, wpt, (int)items, threshold, ws_t, ws_k, flag, out_rgb_dev,          \
                     out_alpha_dev, out_feat_dev)
#define MLPSP_PP_LAUNCH(HT, FT)                 \
  do {                                          \
    if (out_feat_dev) MLPSP_PP_LAUNCH_(HT, FT, true); \
    else MLPSP_PP_LAUNCH_(HT, FT, false);       \
  } while (0)
  if (hidden == 32 && num_frequencies == 6) MLPSP_PP_LAUNCH(32, 6);
  else if (hidden == 16 && num_frequencies == 6) MLPSP_PP_LAUNCH(16, 6);
  else MLPSP_PP_LAUNCH(0, 0);
#undef MLPSP_PP_LAUNCH
#undef MLPSP_PP_LAUNCH_
  MLPSP_LAUNCH_CHECK();
  int32_t host_flag = 0;
  MLPSP_HIP_TRY(hipMemcpyAsync(&host_flag, flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
  MLPSP_HIP_TRY(hipStreamSynchronize(s));
  return host_flag ? MLPSP_E_PIXEL_OVERFLOW : MLPSP_OK;
}

namespace {
template <bool EMIT>
int records_per_pixel_launch(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                             const int32_t* candidates_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                             const float* att_dev, int num_frequencies, const float* W1, const float* b1,
                             const float* W2, const float* b2, const float* W3, const float* b3, int num_primitives,
                             int hidden, float gating_beta, float gating_temp, int width, int height, int tile_w,
                             int tile_h, float threshold, void* workspace_dev, size_t workspace_bytes,
                             int32_t* counts_dev, const int64_t* record_offsets_dev, int32_t* ids_dev, float* x6_dev,
                             int32_t* masks_dev, float* raw_dev, float* gates_dev, float* out_rgb_dev,
                             float* out_alpha_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (num_frequencies <= 0 || num_frequencies > 16 || hidden <= 0 || hidden > 32 || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !workspace_dev) return MLPSP_E_ARGUMENT;
  if (EMIT ? (!record_offsets_dev || !out_rgb_dev || !out_alpha_dev) : !counts_dev) return MLPSP_E_ARGUMENT;
  const size_t need = mlpsp_per_pixel_workspace_bytes(width, height, tile_w, tile_h);
  if (workspace_bytes < need) return MLPSP_E_SCRATCH;
  if (reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  int32_t* flag = reinterpret_cast<int32_t*>(workspace_dev);
  float* ws_t = reinterpret_cast<float*>(static_cast<char*>(workspace_dev) + 256);
  int32_t* ws_k = reinterpret_cast<int32_t*>(ws_t + (size_t)items * 64 * kHitCap);
  MLPSP_HIP_TRY(hipMemsetAsync(flag, 0, sizeof(int32_t), s));
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  MlpPtrs m{W1, b1, W2, b2, W3, b3};
  const dim3 grid((unsigned)items), block(64);
#define MLPSP_RPP_LAUNCH(HT, FT)                                                                                    \
  hipLaunchKernelGGL((records_per_pixel_kernel<HT, FT, EMIT>), grid, block, 0, s, rays_o_dev, rays_d_dev,          \
                     (const PrimRecord*)prim_records_dev, candidates_dev, tile_offsets_dev, freq_dev, att_dev,     \
                     num_frequencies, m, gating_beta, gating_temp, num_primitives, hidden, g, wpt, (int)items,      \
                     threshold, ws_t, ws_k, flag, counts_dev, (const long long*)record_offsets_dev, ids_dev, x6_dev, \
                     masks_dev, raw_dev, gates_dev, out_rgb_dev, out_alpha_dev)
  if (hidden == 32 && num_frequencies == 6) MLPSP_RPP_LAUNCH(32, 6);
  else if (hidden == 16 && num_frequencies == 6) MLPSP_RPP_LAUNCH(16, 6);
  else MLPSP_RPP_LAUNCH(0, 0);
#undef MLPSP_RPP_LAUNCH
  MLPSP_LAUNCH_CHECK();
  int32_t host_flag = 0;
  MLPSP_HIP_TRY(hipMemcpyAsync(&host_flag, flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
  MLPSP_HIP_TRY(hipStreamSynchronize(s));
  return host_flag ? MLPSP_E_PIXEL_OVERFLOW : MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_records_per_pixel_count(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* candidates_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, int width, int height, int tile_w, int tile_h, float threshold,
    void* workspace_dev, size_t workspace_bytes, int32_t* counts_dev, mlpsp_stream_t stream) {
  return records_per_pixel_launch<false>(rays_o_dev, rays_d_dev, prim_records_dev, candidates_dev, tile_offsets_dev,
                                         freq_dev, att_dev, num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives,
                                         hidden, 0.f, 0.f, width, height, tile_w, tile_h, threshold, workspace_dev,
                                         workspace_bytes, counts_dev, nullptr, nullptr, nullptr, nullptr, nullptr,
                                         nullptr, nullptr, nullptr, stream);
}

MLPSP_API int mlpsp_records_per_pixel_emit(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* candidates_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, float gating_beta, float gating_temp, int width, int height, int tile_w,
    int tile_h, float threshold, void* workspace_dev, size_t workspace_bytes, const int64_t* record_offsets_dev,
    int64_t total_records, int32_t* ids_dev, float* x6_dev, int32_t* masks_dev, float* raw_dev, float* gates_dev,
    float* out_rgb_dev, float* out_alpha_dev, mlpsp_stream_t stream) {
  if (total_records < 0) return MLPSP_E_ARGUMENT;
  if (total_records > 0 && (!ids_dev || !x6_dev || !masks_dev || !raw_dev || !gates_dev)) return MLPSP_E_ARGUMENT;
  return records_per_pixel_launch<true>(rays_o_dev, rays_d_dev, prim_records_dev, candidates_dev, tile_offsets_dev,
                                        freq_dev, att_dev, num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives,
                                        hidden, gating_beta, gating_temp, width, height, tile_w, tile_h, threshold,
                                        workspace_dev, workspace_bytes, nullptr, record_offsets_dev, ids_dev, x6_dev,
                                        masks_dev, raw_dev, gates_dev, out_rgb_dev, out_alpha_dev, stream);
}
