// Sum of the rows of a [num_groups, row] f32 matrix per primitive, the groups of primitive p being the
// consecutive rows [group_offsets[p], group_offsets[p+1]) -- the second half of the reference's grouped
// gradient kernels (_reduce_partials, scannet/primitive_gemm.py:169-183; _feature_reduce,
// scannet/record_feature_loss.py:152-161), which give one program per primitive a loop over its groups.
// A frame's records are very unevenly spread (at the 200k-primitive benchmark frame 2,107 primitives share
// 76,600 groups and one of them owns 1,594), so one workgroup per primitive ends in a long tail: 3.3 ms for
// 1 GB of rows.  Here the work is cut by ROWS instead, in two passes with a fixed summation tree:
//   pass 1, one workgroup per chunk of 32 consecutive rows: walk the chunk, summing runs of rows of one
//           primitive.  A run that is the primitive's whole row range goes straight to the output; a run that
//           the next chunk continues goes to tail[chunk]; a run that only continues the previous chunk goes to
//           head[chunk].
//   pass 2, one workgroup per primitive: no rows -> zeros; rows inside one chunk -> nothing to do; otherwise
//           tail[first chunk] + tail[chunks in between] + head[last chunk].
// head/tail are 2 * ceil(num_groups / 32) scratch rows, which the caller provides BEHIND the matrix: the
// buffer holds segment_reduce_rows(num_groups) rows.
#pragma once
#include "mlpsp_host.hpp"

namespace mlpsp {

constexpr int kReduceChunk = 32;

inline int64_t segment_reduce_rows(int64_t num_groups) {
  return num_groups + 2 * ((num_groups + kReduceChunk - 1) / kReduceChunk);
}

// Destination of a primitive's sum: one packed row, or (the MLP gradients) the six tensors whose rows are the
// consecutive parts 2304 | 32 | 1024 | 32 | 128 | 4 of the packed row.
struct ReduceDest {
  float* packed;
  float* part[6];
};

template <int VEC> struct RowVec;
template <> struct RowVec<1> {
  using type = float;
  static __device__ __forceinline__ float zero() { return 0.f; }
  static __device__ __forceinline__ void add(float& a, float b) { a += b; }
  static __device__ __forceinline__ bool bad(float a) { return !(__builtin_fabsf(a) <= 3.4028235e38f); }
};
template <> struct RowVec<4> {
  using type = float4;
  static __device__ __forceinline__ float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void add(float4& a, const float4& b) {
    a.x += b.x;
    a.y += b.y;
    a.z += b.z;
    a.w += b.w;
  }
  static __device__ __forceinline__ bool bad(const float4& a) {
    return !(__builtin_fabsf(a.x) <= 3.4028235e38f) || !(__builtin_fabsf(a.y) <= 3.4028235e38f) ||
           !(__builtin_fabsf(a.z) <= 3.4028235e38f) || !(__builtin_fabsf(a.w) <= 3.4028235e38f);
  }
};

// address of element k (in units of VEC floats) of primitive p's sum
template <int VEC, bool SPLIT>
__device__ __forceinline__ typename RowVec<VEC>::type* reduce_dest(const ReduceDest& d, long long p, int k, int row_vecs) {
  using V = typename RowVec<VEC>::type;
  if constexpr (SPLIT) {
    static_assert(VEC == 4, "the split destination is addressed in float4s");
    // float4 ranges of the parts: [0,576) W1, [576,584) b1, [584,840) W2, [840,848) b2, [848,880) W3, 880 b3
    if (k < 576) return reinterpret_cast<V*>(d.part[0]) + p * 576 + k;
    if (k < 584) return reinterpret_cast<V*>(d.part[1]) + p * 8 + (k - 576);
    if (k < 840) return reinterpret_cast<V*>(d.part[2]) + p * 256 + (k - 584);
    if (k < 848) return reinterpret_cast<V*>(d.part[3]) + p * 8 + (k - 840);
    if (k < 880) return reinterpret_cast<V*>(d.part[4]) + p * 32 + (k - 848);
    return reinterpret_cast<V*>(d.part[5]) + p;
  } else {
    return reinterpret_cast<V*>(d.packed) + p * row_vecs + k;
  }
}

template <int VEC, bool SPLIT>
__global__ __launch_bounds__(256) void segment_reduce_chunks_kernel(
    const float* __restrict__ rows, const long long* __restrict__ group_prim, const long long* __restrict__ group_offsets,
    long long num_groups, int row_vecs, float* __restrict__ scratch, ReduceDest dest, int32_t* __restrict__ nonfinite) {
  using R = RowVec<VEC>;
  using V = typename R::type;
  const long long chunk = blockIdx.x, num_chunks = gridDim.x;
  const long long first = chunk * kReduceChunk;
  const long long last = first + kReduceChunk < num_groups ? first + kReduceChunk : num_groups;
  const V* __restrict__ src = reinterpret_cast<const V*>(rows);
  V* __restrict__ tail = reinterpret_cast<V*>(scratch) + chunk * row_vecs;
  V* __restrict__ head = reinterpret_cast<V*>(scratch) + (num_chunks + chunk) * row_vecs;
  bool bad = false;
  for (int k = threadIdx.x; k < row_vecs; k += 256) {
    V acc = R::zero();
    long long run_start = first, p = group_prim[first];
    for (long long g = first; g <= last; ++g) {
      const long long q = g < last ? group_prim[g] : -1;      // uniform: every thread walks the same rows
      if (q != p) {
        const bool open_start = group_offsets[p] < run_start, open_end = group_offsets[p + 1] > g;
        if (open_end) {
          tail[k] = acc;
        } else if (open_start) {
          head[k] = acc;
        } else {
          *reduce_dest<VEC, SPLIT>(dest, p, k, row_vecs) = acc;
          bad |= R::bad(acc);
        }
        acc = R::zero();
        run_start = g;
        p = q;
      }
      if (g < last) R::add(acc, src[g * row_vecs + k]);
    }
  }
  if (nonfinite && __ballot(bad) != 0ull && (threadIdx.x & 63) == 0) atomicOr(nonfinite, 1);
}

template <int VEC, bool SPLIT>
__global__ __launch_bounds__(256) void segment_reduce_finish_kernel(const long long* __restrict__ group_offsets,
                                                                    long long num_chunks, int row_vecs,
                                                                    const float* __restrict__ scratch, ReduceDest dest,
                                                                    int32_t* __restrict__ nonfinite) {
  using R = RowVec<VEC>;
  using V = typename R::type;
  const long long p = blockIdx.x;
  const long long start = group_offsets[p], end = group_offsets[p + 1];
  if (start < end && start / kReduceChunk == (end - 1) / kReduceChunk) return;      // written by the first pass
  const long long cf = start / kReduceChunk, cl = start < end ? (end - 1) / kReduceChunk : 0;
  const V* __restrict__ tail = reinterpret_cast<const V*>(scratch);
  const V* __restrict__ head = reinterpret_cast<const V*>(scratch) + num_chunks * row_vecs;
  bool bad = false;
  for (int k = threadIdx.x; k < row_vecs; k += 256) {
    V acc = R::zero();
    if (start < end) {
      for (long long c = cf; c < cl; ++c) R::add(acc, tail[c * row_vecs + k]);
      R::add(acc, head[cl * row_vecs + k]);
      bad |= R::bad(acc);
    }
    *reduce_dest<VEC, SPLIT>(dest, p, k, row_vecs) = acc;
  }
  if (nonfinite && __ballot(bad) != 0ull && (threadIdx.x & 63) == 0) atomicOr(nonfinite, 1);
}

// rows_dev: [segment_reduce_rows(num_groups), row_floats]; the first num_groups rows are summed.  The caller has
// cleared nonfinite (it may be null).  SPLIT needs row_floats = 3524.
template <bool SPLIT>
inline int segment_reduce(const float* rows_dev, const int64_t* group_prim_dev, const int64_t* group_offsets_dev,
                          int64_t num_groups, int num_primitives, int64_t row_floats, ReduceDest dest,
                          int32_t* nonfinite_dev, hipStream_t s) {
  if (num_primitives <= 0) return num_primitives < 0 ? MLPSP_E_ARGUMENT : MLPSP_OK;
  if (num_groups < 0 || row_floats <= 0 || row_floats > 2147483647LL || !group_offsets_dev) return MLPSP_E_ARGUMENT;
  if (num_groups > 0 && (!rows_dev || !group_prim_dev)) return MLPSP_E_ARGUMENT;
  uintptr_t bits = reinterpret_cast<uintptr_t>(rows_dev);
  if constexpr (SPLIT) {
    if (row_floats != 3524) return MLPSP_E_ARGUMENT;
    for (float* q : dest.part) {
      if (!q) return MLPSP_E_ARGUMENT;
      bits |= reinterpret_cast<uintptr_t>(q);
    }
    if ((bits & 15) != 0) return MLPSP_E_ARGUMENT;
  } else {
    if (!dest.packed) return MLPSP_E_ARGUMENT;
    bits |= reinterpret_cast<uintptr_t>(dest.packed);
  }
  const long long chunks = (num_groups + kReduceChunk - 1) / kReduceChunk;
  if (chunks > 2147483647LL) return MLPSP_E_ARGUMENT;
  float* scratch = const_cast<float*>(rows_dev) + num_groups * row_floats;
  const bool vec4 = SPLIT || ((row_floats % 4) == 0 && (bits & 15) == 0);
  const dim3 block(256);
#define MLPSP_SEGRED(VEC)                                                                                          \
  do {                                                                                                             \
    const int row_vecs = (int)(row_floats / VEC);                                                                  \
    if (chunks > 0)                                                                                                \
      hipLaunchKernelGGL((segment_reduce_chunks_kernel<VEC, SPLIT>), dim3((unsigned)chunks), block, 0, s, rows_dev, \
                         (const long long*)group_prim_dev, (const long long*)group_offsets_dev,                    \
                         (long long)num_groups, row_vecs, scratch, dest, nonfinite_dev);                           \
    hipLaunchKernelGGL((segment_reduce_finish_kernel<VEC, SPLIT>), dim3((unsigned)num_primitives), block, 0, s,    \
                       (const long long*)group_offsets_dev, chunks, row_vecs, scratch, dest, nonfinite_dev);       \
  } while (0)
  if (vec4) {
    MLPSP_SEGRED(4);
  } else {
    if constexpr (!SPLIT) MLPSP_SEGRED(1);
  }
#undef MLPSP_SEGRED
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

}  // namespace mlpsp
