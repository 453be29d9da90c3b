// libmlpsp_hip: training-records forward (np_tile_kernels.cu:2925-3206 in record modes 1 and 3, wrapper
// :6897-6998): per pixel, one record per hit taken while the pixel is live and below its hit capacity --
// primitive id, MLP input x6, ReLU masks, raw = (R, G, B, sigma_raw, T before the hit, alpha, decay, sigma
// logit) and the four tetrahedral gates -- plus the image composited from those records.  Two launches
// of one kernel: COUNT writes the per-pixel record counts, the caller scans them into offsets, EMIT
// writes the records at offsets[pixel] + k.  Same wave-per-64-pixels traversal as the render kernels.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"
#include "mlpsp_mlp_mfma32.hpp"
#include "mlpsp_render_f32.hpp"
#include "mlpsp_record_stage.hpp"

// records of a pixel staged in LDS before they are written (mlpsp_record_stage.hpp); 8x8 tiles on the matrix-core
// path only -- the scalar shapes keep the direct stores
#ifndef MLPSP_STAGE_K
#define MLPSP_STAGE_K 2
#endif

namespace mlpsp {

struct RecordOut {
  const long long* offsets;   // [B+1] exclusive scan of the counts
  int32_t* ids;               // [R]
  float* x6;                  // [R,6]
  int32_t* masks;             // [R,2]
  float* raw;                 // [R,8]
  float* gates;               // [R,4]
  float* rgb;                 // [B,3]
  float* alpha;               // [B,1]
};

template <bool STAGED> struct F32StageFor { using type = RecordStage<MLPSP_STAGE_K>; };
template <> struct F32StageFor<false> { struct type {}; };

// MF: the MLP of a hit runs on the matrix cores for the whole wavefront (mlp_wave_mfma32, same bits).
// RORD (with MF only): layer 2 in the rounding order of the RENDER kernels instead of the record kernels', so
// that image and records are those of mlpsp_render_tilecenter_f32 bit for bit -- the differentiable render
// then needs no separate forward pass.
template <int HT, int FT, bool EMIT, bool MF = false, bool RORD = false>
__global__ __launch_bounds__(64) void records_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ W2, const float* __restrict__ b2, const float* __restrict__ W3,
    const float* __restrict__ b3, int N, int H, TileGeom g, int waves_per_tile, int per_xcd, int num_items, float thr,
    int max_hits, float beta, float temp, int32_t* __restrict__ counts, int32_t* __restrict__ overflow, RecordOut out) {
  const MlpPtrs mlp{W1, b1, W2, b2, W3, b3};
  const int item = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (item >= num_items) return;
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
  long long rec_base = 0;
  if constexpr (EMIT) rec_base = valid ? out.offsets[pix] : 0;
  // MF kernels run one wavefront per workgroup, which is what the staging needs
  constexpr bool STAGED = EMIT && MF;
  __shared__ typename F32StageFor<STAGED>::type s_stage;
  const RecordArrays arrays{out.ids, out.x6, out.masks, out.raw, out.gates};
  int pending = 0, flushed = 0;
  if constexpr (STAGED) stage_begin(s_stage, (int)threadIdx.x, rdx, rdy, rdz);

  float trans = 1.f, cr = 0.f, cg = 0.f, cb = 0.f;
  int used = 0;
  bool over = false;
  DirOperands dir;
  if constexpr (MF) encode_direction(rdx, rdy, rdz, freq, att, dir);
  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool can = valid && (trans >= kTransmittanceFloor) && (used < max_hits);
    const bool hit = can && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    if (__ballot(hit) != 0ull) {
      const float x6[6] = {rdx, rdy, rdz, hit ? h.dx : 0.f, hit ? h.dy : 0.f, hit ? h.dz : 0.f};
      float o[4];
      uint32_t mk[2];
      if constexpr (MF) mlp_wave_mfma32<!RORD, true>(x6, freq, att, W1, b1, W2, b2, W3, b3, p, dir, o, mk);
      if (hit) {
        if constexpr (!MF) mlp_eval<HT, FT, true>(x6, freq, att, F, H, mlp, p, o, mk);
        const float R = sigmoid(o[0]), G = sigmoid(o[1]), Bc = sigmoid(o[2]);
        const float sigma_raw = softplus(o[3]);
        const float sigma = sigma_raw * h.decay;
        const float alpha = 1.f - det_exp(-sigma);
        if constexpr (EMIT) {
          float gt[4];
          tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
          if constexpr (STAGED) {
            const float rawv[8] = {R, G, Bc, sigma_raw, trans, alpha, h.decay, o[3]};
            stage_put(s_stage, (int)threadIdx.x, pending, p, x6[3], x6[4], x6[5], mk[0], mk[1], rawv, gt);
            ++pending;
          } else {
            const long long r = rec_base + used;
            out.ids[r] = p;
#pragma unroll
            for (int c = 0; c < 6; ++c) out.x6[r * 6 + c] = x6[c];
            out.masks[r * 2] = (int32_t)mk[0];
            out.masks[r * 2 + 1] = (int32_t)mk[1];
            float* __restrict__ raw = out.raw + r * 8;
            raw[0] = R;
            raw[1] = G;
            raw[2] = Bc;
            raw[3] = sigma_raw;
            raw[4] = trans;
            raw[5] = alpha;
            raw[6] = h.decay;
            raw[7] = o[3];
#pragma unroll
            for (int k = 0; k < 4; ++k) out.gates[r * 4 + k] = gt[k];
          }
          const float weight = trans * alpha;
          cr = fmaf(weight, R, cr);
          cg = fmaf(weight, G, cg);
          cb = fmaf(weight, Bc, cb);
        }
        trans = trans * (1.f - alpha);
        ++used;
      }
    }
    if constexpr (STAGED) {
      if (__ballot(pending == MLPSP_STAGE_K) != 0ull) {
        stage_flush(s_stage, (int)threadIdx.x, rec_base + flushed, pending, arrays);
        flushed += pending;
        pending = 0;
      }
    }
    const bool live = valid && (trans >= kTransmittanceFloor);
    over |= live && (used >= max_hits);      // np_tile_kernels.cu:3166-3168: refused, never truncated silently
    if (__ballot(live) == 0ull) break;
  }
  if constexpr (STAGED) {
    if (__ballot(pending > 0) != 0ull) stage_flush(s_stage, (int)threadIdx.x, rec_base + flushed, pending, arrays);
  }
  if (__ballot(over) != 0ull && threadIdx.x == 0) atomicExch(overflow, 1);
  if (valid) {
    if constexpr (EMIT) {
      out.rgb[pix * 3 + 0] = cr;
      out.rgb[pix * 3 + 1] = cg;
      out.rgb[pix * 3 + 2] = cb;
      out.alpha[pix] = 1.f - trans;
    } else {
      counts[pix] = used;
    }
  }
}

}  // namespace mlpsp

using namespace mlpsp;

namespace {
int records_launch(bool emit, const float* rays_o, const float* rays_d, const void* prims, const int32_t* order,
                   const int32_t* offsets, const float* freq, const float* att, int F, const float* W1, const float* b1,
                   const float* W2, const float* b2, const float* W3, const float* b3, int N, int hidden, int width,
                   int height, int tile_w, int tile_h, float thr, int max_hits, int render_order, float beta, float temp,
                   int32_t* counts, int32_t* overflow, RecordOut out, hipStream_t s) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0) return MLPSP_E_ARGUMENT;
  const int64_t tile_px = (int64_t)tile_w * tile_h;
  if (tile_px <= 0 || tile_px > 256) return MLPSP_E_ARGUMENT;
  if (F <= 0 || F > 16 || hidden <= 0 || hidden > 32 || N < 0 || max_hits <= 0) return MLPSP_E_ARGUMENT;
  if (!rays_o || !rays_d || !offsets || !overflow) return MLPSP_E_ARGUMENT;
  if (render_order && !(hidden == 32 && use_mfma32(hidden, F, W1, b1, W2, b2))) return MLPSP_E_ARGUMENT;
  const int wpt = (int)((tile_px + 63) / 64);
  const int64_t items = T * wpt;
  if (items > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  const int per_xcd = (int)((items + kNumXcd - 1) / kNumXcd);
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
#define MLPSP_REC_LAUNCH(HT, FT, ...)                                                                             \
  hipLaunchKernelGGL((records_kernel<HT, FT, ##__VA_ARGS__>), grid, block, 0, s, rays_o, rays_d, (const PrimRecord*)prims,   \
                     order, offsets, freq, att, F, W1, b1, W2, b2, W3, b3, N, hidden, g, wpt, per_xcd, (int)items, \
                     thr, max_hits, beta, temp, counts, overflow, out)
#define MLPSP_REC_SHAPES(EM)                                          \
  do {                                                                \
    if (render_order) MLPSP_REC_LAUNCH(32, 6, EM, true, true);          \
    else if (hidden == 32 && use_mfma32(hidden, F, W1, b1, W2, b2)) MLPSP_REC_LAUNCH(32, 6, EM, true); \
    else if (hidden == 32 && F == 6) MLPSP_REC_LAUNCH(32, 6, EM);     \
    else if (hidden == 16 && F == 6) MLPSP_REC_LAUNCH(16, 6, EM);     \
    else MLPSP_REC_LAUNCH(0, 0, EM);                                  \
  } while (0)
  if (emit) MLPSP_REC_SHAPES(true);
  else MLPSP_REC_SHAPES(false);
#undef MLPSP_REC_SHAPES
#undef MLPSP_REC_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_records_count(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                  const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                  const float* att_dev, int num_frequencies, const float* W1, const float* b1,
                                  const float* W2, const float* b2, const float* W3, const float* b3,
                                  int num_primitives, int hidden, int width, int height, int tile_w, int tile_h,
                                  float threshold, int max_hits, int render_order, int32_t* counts_dev,
                                  int32_t* overflow_dev, mlpsp_stream_t stream) {
  if (!counts_dev || !overflow_dev) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(overflow_dev, 0, sizeof(int32_t), s));
  return records_launch(false, rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,
                        num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives, hidden, width, height, tile_w, tile_h,
                        threshold, max_hits, render_order, 0.f, 0.f, counts_dev, overflow_dev, RecordOut{}, s);
}

MLPSP_API int mlpsp_records_emit(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                 const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                 const float* att_dev, int num_frequencies, const float* W1, const float* b1,
                                 const float* W2, const float* b2, const float* W3, const float* b3,
                                 int num_primitives, int hidden, int width, int height, int tile_w, int tile_h,
                                 float threshold, int max_hits, int render_order, float gating_beta, float gating_temp,
                                 const int64_t* record_offsets_dev, int32_t* ids_dev, float* x6_dev,
                                 int32_t* masks_dev, float* raw_dev, float* gates_dev, float* out_rgb_dev,
                                 float* out_alpha_dev, int32_t* overflow_dev, mlpsp_stream_t stream) {
  if (!record_offsets_dev || !out_rgb_dev || !out_alpha_dev || !overflow_dev) return MLPSP_E_ARGUMENT;
  // the record arrays may be null only when there is nothing to write (the offsets then end at zero)
  RecordOut out{(const long long*)record_offsets_dev, ids_dev, x6_dev, masks_dev, raw_dev, gates_dev, out_rgb_dev,
                out_alpha_dev};
  return records_launch(true, rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,
                        num_frequencies, W1, b1, W2, b2, W3, b3, num_primitives, hidden, width, height, tile_w, tile_h,
                        threshold, max_hits, render_order, gating_beta, gating_temp, nullptr, overflow_dev, out,
                        (hipStream_t)stream);
}
