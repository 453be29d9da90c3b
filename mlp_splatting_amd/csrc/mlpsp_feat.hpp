// Per-hit accumulation of the gated per-primitive feature rows into a chunk of channel accumulators
// (shared by the f32 and the matrix-core feature render kernels).
#pragma once
#include "mlpsp_device.hpp"

namespace mlpsp {

constexpr int kFeatChunk = 128;

// acc[j] += w * mix_j for the chunk's channels; mix as np_tile_kernels.cu:6037-6070.
template <int SLOTS>
__device__ __forceinline__ void feat_chunk_accumulate(float (&acc)[kFeatChunk], const float* __restrict__ rows, int C,
                                                      int nch, float w, const float g[4]) {
#pragma unroll
  for (int j = 0; j < kFeatChunk; ++j) {
    if (j < nch) {
      float mix;
      if constexpr (SLOTS == 1) {
        mix = rows[j];
      } else if constexpr (SLOTS == 4) {
        mix = fmaf(g[0], rows[j], 0.f);
        mix = fmaf(g[1], rows[C + j], mix);
        mix = fmaf(g[2], rows[2 * C + j], mix);
        mix = fmaf(g[3], rows[3 * C + j], mix);
      } else {
        mix = rows[j];
        mix = fmaf(g[0], rows[C + j], mix);
        mix = fmaf(g[1], rows[2 * C + j], mix);
        mix = fmaf(g[2], rows[3 * C + j], mix);
        mix = fmaf(g[3], rows[4 * C + j], mix);
      }
      acc[j] = fmaf(w, mix, acc[j]);
    }
  }
}

// Write one pixel's chunk of accumulators: 16-byte stores when the row layout allows it.
__device__ __forceinline__ void feat_chunk_store(const float (&acc)[kFeatChunk], float* __restrict__ dst, int C, int nch) {
  if ((C & 3) == 0 && (nch & 3) == 0) {
#pragma unroll
    for (int j = 0; j < kFeatChunk; j += 4)
      if (j < nch) *reinterpret_cast<float4*>(dst + j) = make_float4(acc[j], acc[j + 1], acc[j + 2], acc[j + 3]);
  } else {
#pragma unroll
    for (int j = 0; j < kFeatChunk; ++j)
      if (j < nch) dst[j] = acc[j];
  }
}

}  // namespace mlpsp
