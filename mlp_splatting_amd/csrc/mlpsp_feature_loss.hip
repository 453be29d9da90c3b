// libmlpsp_hip: streamed feature L1 loss over saved records and its gradient with respect to the feature
// attributes (counterpart of the reference's Triton kernels _stream_l1, _feature_vjp and _feature_reduce,
// scannet/record_feature_loss.py:12-162).  The high-resolution feature image is never materialised: every
// low-resolution target pixel blends its (up to) four bilinear source pixels from their record lists, and only
// the int8 sign of the residual and a scalar loss partial are kept.  Geometry, alpha and the MLP are constants
// of this loss (:5).
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_segment_reduce.hpp"

namespace mlpsp {

// Feature of one high-resolution pixel and channel from its records: sum_r w_r * mix_r, w = T * alpha,
// mix = base + sum_s gate_s * attr_s (1 slot: attr; 4 slots: gates only; 5 slots: slot 0 is the base)
// (_blend_pixel, record_feature_loss.py:12-31; same fma chain).
template <int SLOTS>
__device__ __forceinline__ float blend_pixel(const int32_t* __restrict__ ids, const long long* __restrict__ offsets,
                                             const float* __restrict__ raw, const float* __restrict__ gates,
                                             const float* __restrict__ attr, long long pixel, int c, int C) {
  float acc = 0.f;
  const long long begin = offsets[pixel], end = offsets[pixel + 1];
  for (long long r = begin; r < end; ++r) {
    const long long p = ids[r];
    const float w = raw[r * 8 + 4] * raw[r * 8 + 5];
    float mix = (SLOTS == 1 || SLOTS == 5) ? attr[p * SLOTS * C + c] : 0.f;
    if constexpr (SLOTS != 1) {
#pragma unroll
      for (int s = 0; s < 4; ++s)
        mix = fmaf(gates[r * 4 + s], attr[(p * SLOTS + s + (SLOTS == 5 ? 1 : 0)) * C + c], mix);
    }
    acc = fmaf(w, mix, acc);
  }
  return acc;
}

// One workgroup = one target pixel x 128 channels (_stream_l1, :34-63).  T = float or _Float16 target.
template <int SLOTS, typename T>
__global__ __launch_bounds__(128) void stream_l1_kernel(const int32_t* __restrict__ ids,
                                                        const long long* __restrict__ offsets,
                                                        const float* __restrict__ raw, const float* __restrict__ gates,
                                                        const float* __restrict__ attr, const T* __restrict__ target,
                                                        int8_t* __restrict__ signs, float* __restrict__ loss,
                                                        float* __restrict__ prediction, int W, int H, int WF, int HF,
                                                        int C) {
  __shared__ float s_part[2];
  const int pix = blockIdx.x, chunk = blockIdx.y;
  const int c = chunk * 128 + threadIdx.x;
  const bool valid = c < C;
  const int cc = valid ? c : 0;
  const float sx = (float)W / (float)WF, sy = (float)H / (float)HF;
  float xf = ((float)(pix % WF) + .5f) * sx - .5f;
  float yf = ((float)(pix / WF) + .5f) * sy - .5f;
  xf = fmaxf(xf, 0.f);
  yf = fmaxf(yf, 0.f);
  const int x0 = (int)xf, y0 = (int)yf;
  const int x1 = min(x0 + 1, W - 1), y1 = min(y0 + 1, H - 1);
  const float wx = xf - (float)x0, wy = yf - (float)y0;
  const float a = blend_pixel<SLOTS>(ids, offsets, raw, gates, attr, (long long)y0 * W + x0, cc, C);
  const float b = blend_pixel<SLOTS>(ids, offsets, raw, gates, attr, (long long)y0 * W + x1, cc, C);
  const float cq = blend_pixel<SLOTS>(ids, offsets, raw, gates, attr, (long long)y1 * W + x0, cc, C);
  const float d = blend_pixel<SLOTS>(ids, offsets, raw, gates, attr, (long long)y1 * W + x1, cc, C);
  const float value = (1.f - wy) * ((1.f - wx) * a + wx * b) + wy * ((1.f - wx) * cq + wx * d);
  const float gt = valid ? (float)target[(long long)pix * C + cc] : 0.f;
  const float delta = value - gt;
  if (valid) {
    signs[(long long)pix * C + c] = (int8_t)((delta > 0.f) - (delta < 0.f));
    if (prediction) prediction[(long long)pix * C + c] = value;
  }
  float part = valid ? __builtin_fabsf(delta) : 0.f;
#pragma unroll
  for (int sft = 1; sft < 64; sft <<= 1) part += __shfl_xor(part, sft);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = part;
  __syncthreads();
  if (threadIdx.x == 0)
    loss[(long long)pix * gridDim.y + chunk] = (s_part[0] + s_part[1]) / (float)((long long)HF * WF * C);
}

// What a record contributes does not depend on the channel except through the signs it samples: its four
// bilinear taps (offset of the target pixel's sign row, weight) and its slot factors T alpha gate_s.  Per batch
// of 64 records these are computed once, lane = record, and parked in LDS; then lane = 4 consecutive channels and
// every record costs four 4-byte sign loads, the tap sums, and a share of a small matrix product (below).
struct RecordTaps {
  int off[4];      // (iy * WF + ix) * C of the tap's target pixel (0 outside the target)
  float weight[4]; // bilinear weight (0 outside the target)
};

typedef _Float16 fh4 __attribute__((ext_vector_type(4)));
typedef float ff4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void record_taps(int pix, int W, int H, int WF, int HF, int C, RecordTaps& t) {
  const int xx = pix % W, yy = pix / W;
  const float fx = (float)WF / (float)W, fy = (float)HF / (float)H, bx = (float)W / (float)WF, by = (float)H / (float)HF;
  const int tx = (int)__builtin_floorf(((float)xx + .5f) * fx - .5f);
  const int ty = (int)__builtin_floorf(((float)yy + .5f) * fy - .5f);
#pragma unroll
  for (int dy = 0; dy < 2; ++dy) {
#pragma unroll
    for (int dx = 0; dx < 2; ++dx) {
      const int ix = tx + dx, iy = ty + dy;
      const float srcx = fmaxf(((float)ix + .5f) * bx - .5f, 0.f);
      const float srcy = fmaxf(((float)iy + .5f) * by - .5f, 0.f);
      const float weight = fmaxf(0.f, 1.f - __builtin_fabsf(srcx - (float)xx)) *
                           fmaxf(0.f, 1.f - __builtin_fabsf(srcy - (float)yy));
      const bool inside = ix >= 0 && ix < WF && iy >= 0 && iy < HF;
      // a tap outside the target reads row 0 with weight 0: the loads of the channel loop need no branch
      t.weight[dy * 2 + dx] = inside ? weight : 0.f;
      t.off[dy * 2 + dx] = inside ? (iy * WF + ix) * C : 0;
    }
  }
}

// One wavefront = one segment of a primitive's records x 256 channels (_feature_vjp, :114-149):
// accum[slot][channel] += (T alpha gate_slot)[record] * adjoint[record's pixel, channel], the adjoint being the
// bilinear transpose of the signs (_resample_adjoint, :92-111: taps added in the order (0,0), (0,1), (1,0),
// (1,1)).  MIXED rounds both factors to fp16 first, as the reference's mixed GEMM does; accumulation is f32.
//
// The sum over records is a [slots x records] x [records x channels] product, and it runs on the matrix cores
// as 4x4 blocks: v_mfma_f32_4x4x4_f16 (mixed; four records per instruction) or v_mfma_f32_4x4x1_f32 (one record,
// an exact f32 fma) treats every group of four lanes as one block, takes from lane l row l%4 of A (a slot's
// factors) and column l%4 of B (the adjoints of ONE of the lane's four channels) and returns to the lane that
// column of the 4x4 result, one slot per register.  One instruction per channel of the lane replaces sixteen
// multiply-adds per record.  Five slots take a second product whose only non-zero row is the fifth slot.
template <int SLOTS, bool MIXED, bool VEC>
__global__ __launch_bounds__(64) void feature_vjp_kernel(const int8_t* __restrict__ signs,
                                                         const long long* __restrict__ order,
                                                         const int32_t* __restrict__ record_pixels,
                                                         const float* __restrict__ raw, const float* __restrict__ gates,
                                                         const long long* __restrict__ offsets,
                                                         const long long* __restrict__ group_prim,
                                                         const long long* __restrict__ group_start,
                                                         const long long* __restrict__ group_order,
                                                         float* __restrict__ partial, int W, int H, int WF, int HF, int C,
                                                         int segment) {
  constexpr int ROWS = SLOTS == 5 ? 8 : 4;                   // slot rows kept in LDS (two products for five slots)
  __shared__ __attribute__((aligned(16))) RecordTaps s_rec[64];
  __shared__ __attribute__((aligned(16))) float s_a[ROWS][64];          // f32 factors, [slot][record]
  __shared__ __attribute__((aligned(8))) _Float16 s_ah[ROWS][64];       // the same rounded to fp16 (mixed)
  // group_order (optional): the segment that workgroup x takes; in the order of the segments' first pixels,
  // workgroups that run together read neighbouring sign rows
  const long long group = group_order ? group_order[blockIdx.x] : (long long)blockIdx.x;
  const int lane = threadIdx.x, m = lane & 3;
  const int c0 = blockIdx.y * 256 + lane * 4;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;
  // VEC (C % 4 == 0): a lane's four channels are one aligned 4-byte load.  Channels past C are clamped to valid
  // addresses and their sums never stored.
  constexpr bool vec = VEC;
  int cc[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) cc[k] = c0 + k < C ? c0 + k : C - 1;
  const int cv = c0 + 3 < C ? c0 : 0;
  ff4 acc[4], acc5[4];                                // [channel of the lane][slot]; acc5[.][0] = fifth slot
#pragma unroll
  for (int k = 0; k < 4; ++k) acc[k] = acc5[k] = ff4{0.f, 0.f, 0.f, 0.f};
  for (long long base = begin; base < end; base += 64) {
    const long long row = base + lane;
    {
      RecordTaps t;
      float a[ROWS];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        t.off[q] = 0;
        t.weight[q] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < ROWS; ++i) a[i] = 0.f;
      if (row < end) {                                  // rows past the end stay empty records: the loop below
        const long long r = order[row];                 // then needs no tail case
        record_taps(record_pixels[r], W, H, WF, HF, C, t);
        const float w = raw[r * 8 + 4] * raw[r * 8 + 5];
#pragma unroll
        for (int sl = 0; sl < SLOTS; ++sl) {
          float g = 1.f;
          if constexpr (SLOTS == 4) g = gates[r * 4 + sl];
          if constexpr (SLOTS == 5) g = (sl == 0) ? 1.f : gates[r * 4 + sl - 1];
          a[sl] = w * g;
        }
      }
      s_rec[lane] = t;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        if constexpr (MIXED) s_ah[i][lane] = (_Float16)a[i];
        else s_a[i][lane] = a[i];
      }
    }
    __syncthreads();
    const int count = (int)((end - base) < 64 ? (end - base) : 64);
    // the sign words of the NEXT four records are requested before the current four are used: with four
    // wavefronts per SIMD the load latency is otherwise paid once per step
    int ahead[16] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (vec) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int tap = 0; tap < 4; ++tap)
          ahead[4 * q + tap] = *reinterpret_cast<const int*>(signs + (long long)s_rec[q].off[tap] + cv);
    }
    for (int rr = 0; rr < count; rr += 4) {
      // adjoints of four records for the lane's four channels
      float bq[4][4];
      int now[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) now[i] = ahead[i];
      if (vec && rr + 4 < count) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int tap = 0; tap < 4; ++tap)
            ahead[4 * q + tap] = *reinterpret_cast<const int*>(signs + (long long)s_rec[rr + 4 + q].off[tap] + cv);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const RecordTaps& t = s_rec[rr + q];
#pragma unroll
        for (int k = 0; k < 4; ++k) bq[q][k] = 0.f;
#pragma unroll
        for (int tap = 0; tap < 4; ++tap) {
          const float wt = t.weight[tap];
          float sv[4];
          if constexpr (vec) {
            const int packed = now[4 * q + tap];
#pragma unroll
            for (int k = 0; k < 4; ++k) sv[k] = (float)(int8_t)(packed >> (8 * k));
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) sv[k] = (float)signs[(long long)t.off[tap] + cc[k]];
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) bq[q][k] = fmaf(wt, sv[k], bq[q][k]);
        }
      }
      if constexpr (MIXED) {
        const fh4 a_op = *reinterpret_cast<const fh4*>(&s_ah[m][rr]);            // rows past the last slot are zero
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const fh4 b_op = {(_Float16)bq[0][k], (_Float16)bq[1][k], (_Float16)bq[2][k], (_Float16)bq[3][k]};
          acc[k] = __builtin_amdgcn_mfma_f32_4x4x4f16(a_op, b_op, acc[k], 0, 0, 0);
          if constexpr (SLOTS == 5) {
            const fh4 a5 = *reinterpret_cast<const fh4*>(&s_ah[4 + m][rr]);       // rows 5..7 are zero
            acc5[k] = __builtin_amdgcn_mfma_f32_4x4x4f16(a5, b_op, acc5[k], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float a_op = s_a[m][rr + q];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            acc[k] = __builtin_amdgcn_mfma_f32_4x4x1f32(a_op, bq[q][k], acc[k], 0, 0, 0);
            if constexpr (SLOTS == 5) acc5[k] = __builtin_amdgcn_mfma_f32_4x4x1f32(s_a[4 + m][rr + q], bq[q][k], acc5[k], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  }
  const float norm = (float)((long long)WF * HF * C);
#pragma unroll
  for (int sl = 0; sl < SLOTS; ++sl)
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (c0 + k < C) partial[(group * SLOTS + sl) * C + c0 + k] = (sl < 4 ? acc[k][sl] : acc5[k][0]) / norm;
}

// Dense adjoint of the feature image (render_tiles_backward_featattr_tilecenter, np_tile_kernels.cu:3531-3760):
// accum[slot][channel] += (T alpha gate_slot)[record] * grad_feat[record's pixel, channel] -- the adjoint of
// the feature image reaches the attributes only, geometry, alpha and gates are constants of it.  The reference
// walks the frame again and adds with atomics in launch order; here the saved records of a primitive are summed
// per segment in record order (f32 fma on the 4x4 matrix-core blocks, as feature_vjp_kernel's exact mode) and the
// segments by the fixed tree of the segmented reduction, so the result does not depend on scheduling.
// One wavefront = one segment x 256 channels; VEC (C % 4 == 0 and a 16-byte aligned image): one load per record.
template <int SLOTS, bool VEC>
__global__ __launch_bounds__(64) void feature_dense_vjp_kernel(const float* __restrict__ grad_feat,
                                                               const long long* __restrict__ order,
                                                               const int32_t* __restrict__ record_pixels,
                                                               const float* __restrict__ raw,
                                                               const float* __restrict__ gates,
                                                               const long long* __restrict__ offsets,
                                                               const long long* __restrict__ group_prim,
                                                               const long long* __restrict__ group_start,
                                                               const long long* __restrict__ group_order,
                                                               float* __restrict__ partial, int C, int segment) {
  constexpr int ROWS = SLOTS == 5 ? 8 : 4;
  __shared__ long long s_row[64];                                       // pixel * C of the staged records
  __shared__ __attribute__((aligned(16))) float s_a[ROWS][64];          // factors, [slot][record]
  // group_order (optional): the segment that workgroup x takes.  Launched in the order of the segments' first
  // pixels, workgroups that run together read neighbouring adjoint rows and share them in L2.
  const long long group = group_order ? group_order[blockIdx.x] : (long long)blockIdx.x;
  const int lane = threadIdx.x, m = lane & 3;
  const int c0 = blockIdx.y * 256 + lane * 4;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;
  int cc[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) cc[k] = c0 + k < C ? c0 + k : C - 1;
  const int cv = c0 + 3 < C ? c0 : 0;
  ff4 acc[4], acc5[4];                                // [channel of the lane][slot]; acc5[.][0] = fifth slot
#pragma unroll
  for (int k = 0; k < 4; ++k) acc[k] = acc5[k] = ff4{0.f, 0.f, 0.f, 0.f};
  auto fetch = [&](int rec, float (&v)[4]) {
    const float* __restrict__ src = grad_feat + s_row[rec];
    if constexpr (VEC) {
      const float4 q = *reinterpret_cast<const float4*>(src + cv);
      v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = src[cc[k]];
    }
  };
  for (long long base = begin; base < end; base += 64) {
    const long long row = base + lane;
    {
      float a[ROWS];
#pragma unroll
      for (int i = 0; i < ROWS; ++i) a[i] = 0.f;
      long long pixel_row = 0;
      if (row < end) {
        const long long r = order[row];
        pixel_row = (long long)record_pixels[r] * C;
        const float w = raw[r * 8 + 4] * raw[r * 8 + 5];
#pragma unroll
        for (int sl = 0; sl < SLOTS; ++sl) {
          float g = 1.f;
          if constexpr (SLOTS == 4) g = gates[r * 4 + sl];
          if constexpr (SLOTS == 5) g = (sl == 0) ? 1.f : gates[r * 4 + sl - 1];
          a[sl] = w * g;
        }
      }
      s_row[lane] = pixel_row;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) s_a[i][lane] = a[i];
    }
    __syncthreads();
    const int count = (int)((end - base) < 64 ? (end - base) : 64);
    // the adjoint rows of the NEXT four records are requested before the current four are used
    float ahead[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q) fetch(q, ahead[q]);
    for (int rr = 0; rr < count; rr += 4) {
      float now[4][4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int k = 0; k < 4; ++k) now[q][k] = (rr + q < count) ? ahead[q][k] : 0.f;   // an empty record adds +0
      if (rr + 4 < count) {
#pragma unroll
        for (int q = 0; q < 4; ++q) fetch(rr + 4 + q, ahead[q]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float a_op = s_a[m][rr + q];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          acc[k] = __builtin_amdgcn_mfma_f32_4x4x1f32(a_op, now[q][k], acc[k], 0, 0, 0);
          if constexpr (SLOTS == 5)
            acc5[k] = __builtin_amdgcn_mfma_f32_4x4x1f32(s_a[4 + m][rr + q], now[q][k], acc5[k], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int sl = 0; sl < SLOTS; ++sl)
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (c0 + k < C) partial[(group * SLOTS + sl) * C + c0 + k] = sl < 4 ? acc[k][sl] : acc5[k][0];
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_stream_feature_l1(const int32_t* ids_dev, const int64_t* pixel_offsets_dev, const float* raw_dev,
                                      const float* gates_dev, const float* attributes_dev, const void* target_dev,
                                      int target_is_half, int width, int height, int target_width, int target_height,
                                      int channels, int slots, int8_t* signs_dev, float* loss_partials_dev,
                                      float* prediction_dev, mlpsp_stream_t stream) {
  if (width <= 0 || height <= 0 || target_width <= 0 || target_height <= 0 || channels <= 0) return MLPSP_E_ARGUMENT;
  if (target_width > width || target_height > height) return MLPSP_E_ARGUMENT;
  if (slots != 1 && slots != 4 && slots != 5) return MLPSP_E_ARGUMENT;
  if ((int64_t)target_width * target_height > 2147483647LL) return MLPSP_E_ARGUMENT;
  if (!pixel_offsets_dev || !attributes_dev || !target_dev || !signs_dev || !loss_partials_dev) return MLPSP_E_ARGUMENT;
  const dim3 grid((unsigned)(target_width * target_height), (unsigned)((channels + 127) / 128)), block(128);
  hipStream_t s = (hipStream_t)stream;
#define MLPSP_L1_LAUNCH(SL, T)                                                                                     \
  hipLaunchKernelGGL((stream_l1_kernel<SL, T>), grid, block, 0, s, ids_dev, (const long long*)pixel_offsets_dev,   \
                     raw_dev, gates_dev, attributes_dev, (const T*)target_dev, signs_dev, loss_partials_dev,       \
                     prediction_dev, width, height, target_width, target_height, channels)
#define MLPSP_L1_SLOTS(T)                         \
  do {                                            \
    if (slots == 1) MLPSP_L1_LAUNCH(1, T);        \
    else if (slots == 4) MLPSP_L1_LAUNCH(4, T);   \
    else MLPSP_L1_LAUNCH(5, T);                   \
  } while (0)
  if (target_is_half) MLPSP_L1_SLOTS(_Float16);
  else MLPSP_L1_SLOTS(float);
#undef MLPSP_L1_SLOTS
#undef MLPSP_L1_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_feature_attribute_gradients(const int8_t* signs_dev, const int64_t* record_indices_dev,
                                                const int32_t* record_pixels_dev, const float* raw_dev,
                                                const float* gates_dev, const int64_t* csr_offsets_dev,
                                                const int64_t* group_primitives_dev, const int64_t* group_starts_dev,
                                                const int64_t* group_offsets_dev, const int64_t* group_order_dev,
                                                int64_t num_groups, int num_primitives, int width, int height,
                                                int target_width,
                                                int target_height, int channels, int slots, int segment, int mixed,
                                                float* partial_dev, float* out_dev, mlpsp_stream_t stream) {
  if (width <= 0 || height <= 0 || target_width <= 0 || target_height <= 0 || channels <= 0 || segment <= 0)
    return MLPSP_E_ARGUMENT;
  if (target_width > width || target_height > height || num_groups < 0 || num_groups > 2147483647LL ||
      num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (slots != 1 && slots != 4 && slots != 5) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (num_groups > 0) {
    if (!signs_dev || !record_indices_dev || !record_pixels_dev || !raw_dev || !csr_offsets_dev ||
        !group_primitives_dev || !group_starts_dev || !partial_dev)
      return MLPSP_E_ARGUMENT;
    const dim3 grid((unsigned)num_groups, (unsigned)((channels + 255) / 256)), block(64);
#define MLPSP_FV_LAUNCH(SL, MX, VC)                                                                                \
  hipLaunchKernelGGL((feature_vjp_kernel<SL, MX, VC>), grid, block, 0, s, signs_dev,                               \
                     (const long long*)record_indices_dev, record_pixels_dev, raw_dev, gates_dev,                  \
                     (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,                    \
                     (const long long*)group_starts_dev, (const long long*)group_order_dev, partial_dev, width,    \
                     height, target_width, target_height, channels, segment)
#define MLPSP_FV_SLOTS(MX, VC)                         \
  do {                                                 \
    if (slots == 1) MLPSP_FV_LAUNCH(1, MX, VC);        \
    else if (slots == 4) MLPSP_FV_LAUNCH(4, MX, VC);   \
    else MLPSP_FV_LAUNCH(5, MX, VC);                   \
  } while (0)
    const bool aligned4 = (channels % 4 == 0) && (reinterpret_cast<uintptr_t>(signs_dev) % 4 == 0);
    if (mixed) {
      if (aligned4) MLPSP_FV_SLOTS(true, true);
      else MLPSP_FV_SLOTS(true, false);
    } else {
      if (aligned4) MLPSP_FV_SLOTS(false, true);
      else MLPSP_FV_SLOTS(false, false);
    }
#undef MLPSP_FV_SLOTS
#undef MLPSP_FV_LAUNCH
    MLPSP_LAUNCH_CHECK();
  }
  // out[p] = sum over the primitive's segments (_feature_reduce, :152-161)
  if (num_primitives > 0) {
    ReduceDest dest{};
    dest.packed = out_dev;
    const int rc = segment_reduce<false>(partial_dev, group_primitives_dev, group_offsets_dev, num_groups, num_primitives,
                                         (int64_t)slots * channels, dest, nullptr, s);
    if (rc != MLPSP_OK) return rc;
  }
  return MLPSP_OK;
}

MLPSP_API int mlpsp_feature_dense_attribute_gradients(const float* grad_feat_dev, const int64_t* record_indices_dev,
                                                      const int32_t* record_pixels_dev, const float* raw_dev,
                                                      const float* gates_dev, const int64_t* csr_offsets_dev,
                                                      const int64_t* group_primitives_dev,
                                                      const int64_t* group_starts_dev, const int64_t* group_offsets_dev,
                                                      const int64_t* group_order_dev, int64_t num_groups,
                                                      int num_primitives, int channels, int slots,
                                                      int segment, float* partial_dev, float* out_dev,
                                                      mlpsp_stream_t stream) {
  if (channels <= 0 || segment <= 0 || num_groups < 0 || num_groups > 2147483647LL || num_primitives < 0)
    return MLPSP_E_ARGUMENT;
  if (slots != 1 && slots != 4 && slots != 5) return MLPSP_E_ARGUMENT;
  if (slots != 1 && num_groups > 0 && !gates_dev) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (num_groups > 0) {
    if (!grad_feat_dev || !record_indices_dev || !record_pixels_dev || !raw_dev || !csr_offsets_dev ||
        !group_primitives_dev || !group_starts_dev || !partial_dev)
      return MLPSP_E_ARGUMENT;
    const dim3 grid((unsigned)num_groups, (unsigned)((channels + 255) / 256)), block(64);
#define MLPSP_FD_LAUNCH(SL, VC)                                                                                    \
  hipLaunchKernelGGL((feature_dense_vjp_kernel<SL, VC>), grid, block, 0, s, grad_feat_dev,                         \
                     (const long long*)record_indices_dev, record_pixels_dev, raw_dev, gates_dev,                  \
                     (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,                    \
                     (const long long*)group_starts_dev, (const long long*)group_order_dev, partial_dev, channels,  \
                     segment)
#define MLPSP_FD_SLOTS(VC)                         \
  do {                                             \
    if (slots == 1) MLPSP_FD_LAUNCH(1, VC);        \
    else if (slots == 4) MLPSP_FD_LAUNCH(4, VC);   \
    else MLPSP_FD_LAUNCH(5, VC);                   \
  } while (0)
    if ((channels % 4 == 0) && (reinterpret_cast<uintptr_t>(grad_feat_dev) % 16 == 0)) MLPSP_FD_SLOTS(true);
    else MLPSP_FD_SLOTS(false);
#undef MLPSP_FD_SLOTS
#undef MLPSP_FD_LAUNCH
    MLPSP_LAUNCH_CHECK();
  }
  if (num_primitives > 0) {
    ReduceDest dest{};
    dest.packed = out_dev;
    const int rc = segment_reduce<false>(partial_dev, group_primitives_dev, group_offsets_dev, num_groups, num_primitives,
                                         (int64_t)slots * channels, dest, nullptr, s);
    if (rc != MLPSP_OK) return rc;
  }
  return MLPSP_OK;
}
