// libmlpsp_hip: training-records forward with the 72->32->32->4 MLP on the matrix cores.
//
// Counterpart of the reference's opt-in mixed-precision record forward (scannet/cuda/training_wmma.cuh:62-253):
// the records of mlpsp_records.hip -- per pixel and hit the primitive id, the MLP input x6, the ReLU masks,
// raw = (R, G, B, sigma_raw, T before the hit, alpha, decay, sigma logit) and the tetrahedral gates, plus the
// image composited from them -- with geometry, ordering, gates, activations and compositing in the same f32
// expressions as the scalar record forward (ids, x6, decay, gates and, while the hit sets agree, the offsets
// are bit-identical to it), and only the MLP in fp16/bf16 operands with f32 accumulation
// (mlp_wave_mfma16).  Differences from the reference's kernel, both inside its stated tolerances: the biases
// of the hidden layers enter as the accumulators' initial value instead of being added after the product,
// and a unit counts as active in the saved masks when its ROUNDED activation -- the value the next layer
// really multiplies -- is non-zero (the reference tests the f32 pre-activation; the two differ only for fp16
// values below 2^-25).
//
// Two launches of ONE kernel with a run-time emit flag's worth of difference only in what is stored (COUNT
// writes per-pixel counts, EMIT writes the records at offsets[pixel] + k and the image): both passes execute
// the same arithmetic, so their hit sets agree; EMIT nevertheless guards every write by the pixel's own
// interval and reports a disagreement instead of writing outside it (training_wmma.cuh:140-147, 224-236).
// status bits: 1 numeric (non-finite operand, activation or output -- the caller repeats the frame in f32),
// 2 hit capacity, 4 count/emit disagreement.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mfma16.hpp"
#include "mlpsp_record_stage.hpp"

// records of a pixel staged in LDS before they are written (mlpsp_record_stage.hpp)
#ifndef MLPSP_STAGE_K
#define MLPSP_STAGE_K 2
#endif

namespace mlpsp {

constexpr int kStatusNumeric = 1, kStatusCapacity = 2, kStatusMismatch = 4;

struct MixedRecordOut {
  const long long* offsets;   // [B+1] exclusive scan of the counts
  long long total;            // offsets[B]
  int32_t* ids;               // [R]
  float* x6;                  // [R,6]
  int32_t* masks;             // [R,2]
  float* raw;                 // [R,8]
  float* gates;               // [R,4]
  float* rgb;                 // [B,3]
  float* alpha;               // [B,1]
};

__device__ __forceinline__ bool not_finite(float v) { return !(__builtin_fabsf(v) <= 3.4028235e38f); }

template <bool EMIT> struct StageFor { using type = RecordStage<MLPSP_STAGE_K>; };
template <> struct StageFor<false> { struct type {}; };

// One read-only pass over up to 16 f32 arrays; flag[0] |= 1 if any element is NaN or infinite
// (training_wmma.cuh:24-60: one fused scan and one read-back instead of a reduction per tensor).
struct FiniteScanInputs {
  const float* pointers[16];
  long long lengths[16];
  int count;
};

__global__ __launch_bounds__(256) void finite_scan_kernel(FiniteScanInputs in, int32_t* __restrict__ flag) {
  bool bad = false;
  const long long stride = (long long)blockDim.x * gridDim.x, first = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  for (int t = 0; t < in.count; ++t) {
    const float* __restrict__ src = in.pointers[t];
    const long long n = in.lengths[t];
    // 16-byte loads over the aligned middle, scalar loads for the ragged ends
    const long long head = min(n, (long long)(((16 - (reinterpret_cast<uintptr_t>(src) & 15)) & 15) / 4));
    const long long quads = (n - head) / 4;
    const f32x4* __restrict__ mid = reinterpret_cast<const f32x4*>(src + head);
    for (long long i = first; i < quads; i += stride) {
      const f32x4 v = mid[i];
      bad |= not_finite(v[0]) || not_finite(v[1]) || not_finite(v[2]) || not_finite(v[3]);
    }
    for (long long i = first; i < head; i += stride) bad |= not_finite(src[i]);
    for (long long i = head + 4 * quads + first; i < n; i += stride) bad |= not_finite(src[i]);
  }
  if (__ballot(bad) != 0ull && (threadIdx.x & 63) == 0) atomicOr(flag, 1);
}

template <typename T, bool EMIT>
__device__ __forceinline__ void records_mfma_body(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, const unsigned char* __restrict__ packed, int N, int W, int H, int ntx, int per_xcd,
    int num_tiles, float thr, int max_hits, float beta, float temp, int32_t* __restrict__ counts,
    int32_t* __restrict__ status, const MixedRecordOut& out) {
  const int tile = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (tile >= num_tiles) return;
  const int l = threadIdx.x;
  float kf[3];
  phase_scales(freq, att, l >> 5, kf);
  const int tx = tile % ntx, ty = tile / ntx;
  const int x = tx * 8 + (l & 7), y = ty * 8 + (l >> 3);
  const bool valid = (x < W) && (y < H);
  const int pix = valid ? (y * W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f, roy = valid ? rays_o[pix * 3 + 1] : 0.f,
              roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f, rdy = valid ? rays_d[pix * 3 + 1] : 0.f,
              rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  __shared__ DirWords s_dir;
  encode_direction_words<T>(rdx, rdy, rdz, kf, l, s_dir);

  long long rec_base = 0;
  int expected = 0, pending = 0, flushed = 0;
  bool mismatch = false;
  __shared__ typename StageFor<EMIT>::type s_stage;
  const RecordArrays arrays{out.ids, out.x6, out.masks, out.raw, out.gates};
  if constexpr (EMIT) {
    stage_begin(s_stage, l, rdx, rdy, rdz);
    if (valid) {
      rec_base = out.offsets[pix];
      const long long rec_end = out.offsets[pix + 1];
      const bool range_ok = rec_base >= 0 && rec_end >= rec_base && rec_end <= out.total && rec_end - rec_base <= max_hits;
      mismatch = !range_ok;
      expected = range_ok ? (int)(rec_end - rec_base) : 0;
    }
  }

  const int start = offsets[tile], end = offsets[tile + 1];
  float trans = 1.f, cr = 0.f, cg = 0.f, cb = 0.f;
  int used = 0;
  bool over = false, bad = false;
  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool can = valid && (trans >= kTransmittanceFloor) && (used < max_hits);
    const bool hit = can && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    const unsigned long long mask = __ballot(hit);
    if (mask != 0ull) {
      const unsigned char* __restrict__ blk = packed + (size_t)p * kPackStride;
      const float dx = hit ? h.dx : 0.f, dy = hit ? h.dy : 0.f, dz = hit ? h.dz : 0.f;
      bad |= hit && (not_finite((dx + dy) + dz) || not_finite(h.decay));
      float o[4];
      unsigned mk[2] = {0u, 0u};
      bad |= mlp_wave_mfma16<T, true, EMIT>(blk, mask, l, dx, dy, dz, kf, s_dir, o, mk);
      if (hit) {
        const float R = sigmoid(o[0]), G = sigmoid(o[1]), Bc = sigmoid(o[2]);
        const float sigma_raw = softplus(o[3]);
        const float sigma = sigma_raw * h.decay;
        const float alpha = 1.f - det_exp(-sigma);
        bad |= not_finite((o[0] + o[1]) + (o[2] + o[3])) || not_finite((R + G) + (Bc + sigma_raw)) || not_finite(alpha);
        if constexpr (EMIT) {
          if (used < expected) {
            const float rawv[8] = {R, G, Bc, sigma_raw, trans, alpha, h.decay, o[3]};
            float gt[4];
            tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
            bad |= not_finite((gt[0] + gt[1]) + (gt[2] + gt[3]));
            stage_put(s_stage, l, pending, p, dx, dy, dz, mk[0], mk[1], rawv, gt);
            ++pending;
          } else {
            mismatch = true;
          }
          const float weight = trans * alpha;
          cr = fmaf(weight, R, cr);
          cg = fmaf(weight, G, cg);
          cb = fmaf(weight, Bc, cb);
        }
        trans = trans * (1.f - alpha);
        ++used;
        bad |= not_finite(trans);
      }
    }
    if constexpr (EMIT) {
      // a pixel's interval holds `expected` records and `flushed + pending` never exceeds it
      if (__ballot(pending == MLPSP_STAGE_K) != 0ull) {
        stage_flush(s_stage, l, rec_base + flushed, pending, arrays);
        flushed += pending;
        pending = 0;
      }
    }
    const bool live = valid && (trans >= kTransmittanceFloor);
    over |= live && (used >= max_hits);      // refused, never truncated silently (training_wmma.cuh:243-244)
    if (__ballot(live) == 0ull) break;
  }
  if constexpr (EMIT) {
    if (__ballot(pending > 0) != 0ull) stage_flush(s_stage, l, rec_base + flushed, pending, arrays);
    mismatch |= valid && (used != expected);
    bad |= not_finite((cr + cg) + cb);
  }
  int bits = 0;
  if (__ballot(bad) != 0ull) bits |= kStatusNumeric;
  if (__ballot(over) != 0ull) bits |= kStatusCapacity;
  if (__ballot(mismatch) != 0ull) bits |= kStatusMismatch;
  if (bits != 0 && l == 0) atomicOr(status, bits);
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

#define MLPSP_RECM_PARAMS                                                                                              \
  const float *__restrict__ rays_o, const float *__restrict__ rays_d, const PrimRecord *__restrict__ prims,            \
      const int32_t *__restrict__ order, const int32_t *__restrict__ offsets, const float *__restrict__ freq,          \
      const float *__restrict__ att, const unsigned char *__restrict__ packed, int N, int W, int H, int ntx,           \
      int per_xcd, int num_tiles, float thr, int max_hits, float beta, float temp, int32_t *__restrict__ counts,       \
      int32_t *__restrict__ status, MixedRecordOut out
#define MLPSP_RECM_ARGS                                                                                                \
  rays_o, rays_d, prims, order, offsets, freq, att, packed, N, W, H, ntx, per_xcd, num_tiles, thr, max_hits, beta,     \
      temp, counts, status, out

// The count pass fits 128 registers without spilling: four wavefronts per SIMD (measured 1.19 -> 1.12 ms at
// 200k primitives).  The emit pass does not (capped at 128 it spills and measured slower), and its staging area
// limits it to two wavefronts per SIMD; staged stores still win: 3.6 -> 3.0 ms, HBM writes 7.0 -> 4.2 GB and
// re-fetched weights 2.9 -> 1.0 GB per launch (K = 4 measures the same as K = 2 and holds more LDS).
template <typename T>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 4))) void records_mfma_count_kernel(MLPSP_RECM_PARAMS) {
  records_mfma_body<T, false>(MLPSP_RECM_ARGS);
}
template <typename T>
__global__ __launch_bounds__(64) void records_mfma_emit_kernel(MLPSP_RECM_PARAMS) {
  records_mfma_body<T, true>(MLPSP_RECM_ARGS);
}
#undef MLPSP_RECM_PARAMS
#undef MLPSP_RECM_ARGS

}  // namespace mlpsp

using namespace mlpsp;

namespace {
int records_mfma_launch(bool emit, const float* rays_o, const float* rays_d, const void* prims, const int32_t* order,
                        const int32_t* offsets, const float* freq, const float* att, const void* packed, int N, int width,
                        int height, float thr, int max_hits, int bf16, float beta, float temp, int32_t* counts,
                        int32_t* status, MixedRecordOut out, hipStream_t s) {
  const int64_t T = checked_num_tiles(width, height, 8, 8);
  if (T <= 0 || T > 2147483647LL - 8) return MLPSP_E_ARGUMENT;
  if (N < 0 || max_hits <= 0 || !(thr > 0.f && thr < 1.f)) return MLPSP_E_ARGUMENT;
  if (!rays_o || !rays_d || !offsets || !status || !freq || !att) return MLPSP_E_ARGUMENT;
  if (N > 0 && (!prims || !packed)) return MLPSP_E_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(prims) % 128) != 0 || (reinterpret_cast<uintptr_t>(packed) % 16) != 0)
    return MLPSP_E_ARGUMENT;
  const int per_xcd = (int)((T + kNumXcd - 1) / kNumXcd);
  const int ntx = ceil_div(width, 8);
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
#define MLPSP_RECM_LAUNCH(KERNEL)                                                                                    \
  hipLaunchKernelGGL(KERNEL, grid, block, 0, s, rays_o, rays_d, (const PrimRecord*)prims, order, offsets, freq, att,   \
                     (const unsigned char*)packed, N, width, height, ntx, per_xcd, (int)T, thr, max_hits, beta, temp,  \
                     counts, status, out)
  if (bf16) {
    if (emit) MLPSP_RECM_LAUNCH(records_mfma_emit_kernel<__bf16>);
    else MLPSP_RECM_LAUNCH(records_mfma_count_kernel<__bf16>);
  } else {
    if (emit) MLPSP_RECM_LAUNCH(records_mfma_emit_kernel<_Float16>);
    else MLPSP_RECM_LAUNCH(records_mfma_count_kernel<_Float16>);
  }
#undef MLPSP_RECM_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_records_mfma_count(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                       const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                       const float* att_dev, const void* packed_dev, int num_primitives, int width,
                                       int height, float threshold, int max_hits, int bf16, int32_t* counts_dev,
                                       int32_t* status_dev, mlpsp_stream_t stream) {
  if (!counts_dev) return MLPSP_E_ARGUMENT;
  return records_mfma_launch(false, rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, freq_dev,
                             att_dev, packed_dev, num_primitives, width, height, threshold, max_hits, bf16, 0.f, 0.f,
                             counts_dev, status_dev, MixedRecordOut{}, (hipStream_t)stream);
}

MLPSP_API int mlpsp_records_mfma_emit(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                      const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                      const float* att_dev, const void* packed_dev, int num_primitives, int width,
                                      int height, float threshold, int max_hits, int bf16, float gating_beta,
                                      float gating_temp, const int64_t* record_offsets_dev, int64_t total_records,
                                      int32_t* ids_dev, float* x6_dev, int32_t* masks_dev, float* raw_dev,
                                      float* gates_dev, float* out_rgb_dev, float* out_alpha_dev, int32_t* status_dev,
                                      mlpsp_stream_t stream) {
  if (!record_offsets_dev || !out_rgb_dev || !out_alpha_dev || total_records < 0) return MLPSP_E_ARGUMENT;
  if (total_records > 0 && (!ids_dev || !x6_dev || !masks_dev || !raw_dev || !gates_dev)) return MLPSP_E_ARGUMENT;
  MixedRecordOut out{(const long long*)record_offsets_dev, (long long)total_records, ids_dev, x6_dev, masks_dev,
                     raw_dev,  gates_dev, out_rgb_dev, out_alpha_dev};
  return records_mfma_launch(true, rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, freq_dev,
                             att_dev, packed_dev, num_primitives, width, height, threshold, max_hits, bf16, gating_beta,
                             gating_temp, nullptr, status_dev, out, (hipStream_t)stream);
}

MLPSP_API int mlpsp_all_finite(const float* const* arrays_dev, const int64_t* lengths, int num_arrays, int32_t* flag_dev,
                               mlpsp_stream_t stream) {
  if (num_arrays < 0 || num_arrays > 16 || !flag_dev || (num_arrays > 0 && (!arrays_dev || !lengths)))
    return MLPSP_E_ARGUMENT;
  FiniteScanInputs in{};
  long long largest = 0;
  for (int t = 0; t < num_arrays; ++t) {
    if (lengths[t] < 0 || (lengths[t] > 0 && !arrays_dev[t])) return MLPSP_E_ARGUMENT;
    if (lengths[t] == 0) continue;
    if ((reinterpret_cast<uintptr_t>(arrays_dev[t]) & 3) != 0) return MLPSP_E_ARGUMENT;
    in.pointers[in.count] = arrays_dev[t];
    in.lengths[in.count] = lengths[t];
    largest = lengths[t] > largest ? lengths[t] : largest;
    ++in.count;
  }
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(flag_dev, 0, sizeof(int32_t), s));
  if (in.count == 0) return MLPSP_OK;
  const long long want = (largest / 4 + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : (want > 8192 ? 8192 : want));
  hipLaunchKernelGGL(finite_scan_kernel, dim3(blocks), dim3(256), 0, s, in, flag_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
