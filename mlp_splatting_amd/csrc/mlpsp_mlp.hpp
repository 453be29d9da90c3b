// Scalar f32 evaluation of one primitive's light-field MLP (shared by the f32 render kernels).
#pragma once
#include "mlpsp_device.hpp"

namespace mlpsp {

struct MlpPtrs {
  const float *W1, *b1, *W2, *b2, *W3, *b3;
};

// Fixed-shape MLP, fully unrolled: activations live in VGPRs, weights arrive as scalar operands.
// Accumulation order per hidden unit is that of np_tile_kernels.cu:2050-2089: start from the bias,
// then for j = c*F+f ascending add W1[h][j]*sin_j and W1[h][j+6F]*cos_j.
//
// REC selects the arithmetic of the record kernels (mlp_eval_rgb_sigma, np_tile_kernels.cu:313-381): layer 2 is
// bias + (fma chain started at zero) there, which rounds differently from the chain started at the bias,
// and masks[l] receives bit h iff hidden unit h of layer l+1 is positive (:371-379).
template <int H, int F, bool REC = false>
__device__ __forceinline__ void mlp_fixed(const float x6[6], const float* __restrict__ freq,
                                          const float* __restrict__ att, const MlpPtrs& m, int p, float out[4],
                                          uint32_t* masks = nullptr) {
  constexpr int IN = 12 * F, HALF = 6 * F;
  float sn[HALF], cs[HALF];
#pragma unroll
  for (int c = 0; c < 6; ++c) {
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const float phase = (x6[c] * freq[f]) * att[f];
      det_sincos(phase, sn[c * F + f], cs[c * F + f]);
    }
  }
  const float* __restrict__ w1 = m.W1 + (size_t)p * (H * IN);
  const float* __restrict__ bb1 = m.b1 + (size_t)p * H;
  const float* __restrict__ w2 = m.W2 + (size_t)p * (H * H);
  const float* __restrict__ bb2 = m.b2 + (size_t)p * H;
  const float* __restrict__ w3 = m.W3 + (size_t)p * (4 * H);
  const float* __restrict__ bb3 = m.b3 + (size_t)p * 4;
  float h1[H], h2[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    float acc = bb1[h];
#pragma unroll
    for (int j = 0; j < HALF; ++j) {
      acc = fmaf(w1[h * IN + j], sn[j], acc);
      acc = fmaf(w1[h * IN + HALF + j], cs[j], acc);
    }
    h1[h] = acc > 0.f ? acc : 0.f;
  }
#pragma unroll
  for (int o = 0; o < H; ++o) {
    float acc = REC ? 0.f : bb2[o];
#pragma unroll
    for (int h = 0; h < H; ++h) acc = fmaf(w2[o * H + h], h1[h], acc);
    if constexpr (REC) acc = bb2[o] + acc;
    h2[o] = acc > 0.f ? acc : 0.f;
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float acc = bb3[k];
#pragma unroll
    for (int h = 0; h < H; ++h) acc = fmaf(w3[k * H + h], h2[h], acc);
    out[k] = acc;
  }
  if constexpr (REC) {
    uint32_t m1 = 0u, m2 = 0u;
#pragma unroll
    for (int h = 0; h < H && h < 32; ++h) {
      m1 |= (h1[h] > 0.f) ? (1u << h) : 0u;
      m2 |= (h2[h] > 0.f) ? (1u << h) : 0u;
    }
    masks[0] = m1;
    masks[1] = m2;
  }
}

// Any H <= 64, F <= 16: same order, run-time loops (activations spill to scratch; used for the
// odd shapes only).
template <bool REC = false>
static __device__ __noinline__ void mlp_generic(const float x6[6], const float* __restrict__ freq,
                                         const float* __restrict__ att, int F, int H, const MlpPtrs& m, int p,
                                         float out[4], uint32_t* masks = nullptr) {
  const int IN = 12 * F, HALF = 6 * F;
  float h1[64], h2[64];
  const float* w1 = m.W1 + (size_t)p * H * IN;
  const float* bb1 = m.b1 + (size_t)p * H;
  const float* w2 = m.W2 + (size_t)p * H * H;
  const float* bb2 = m.b2 + (size_t)p * H;
  const float* w3 = m.W3 + (size_t)p * 4 * H;
  const float* bb3 = m.b3 + (size_t)p * 4;
  for (int h = 0; h < H; ++h) h1[h] = bb1[h];
  for (int c = 0; c < 6; ++c) {
    for (int f = 0; f < F; ++f) {
      float s, co;
      det_sincos((x6[c] * freq[f]) * att[f], s, co);
      const int j = c * F + f;
      for (int h = 0; h < H; ++h) {
        h1[h] = fmaf(w1[h * IN + j], s, h1[h]);
        h1[h] = fmaf(w1[h * IN + HALF + j], co, h1[h]);
      }
    }
  }
  for (int h = 0; h < H; ++h) h1[h] = h1[h] > 0.f ? h1[h] : 0.f;
  for (int o = 0; o < H; ++o) {
    float acc = REC ? 0.f : bb2[o];
    for (int h = 0; h < H; ++h) acc = fmaf(w2[o * H + h], h1[h], acc);
    if constexpr (REC) acc = bb2[o] + acc;
    h2[o] = acc > 0.f ? acc : 0.f;
  }
  for (int k = 0; k < 4; ++k) {
    float acc = bb3[k];
    for (int h = 0; h < H; ++h) acc = fmaf(w3[k * H + h], h2[h], acc);
    out[k] = acc;
  }
  if constexpr (REC) {
    uint32_t m1 = 0u, m2 = 0u;
    for (int h = 0; h < H && h < 32; ++h) {
      m1 |= (h1[h] > 0.f) ? (1u << h) : 0u;
      m2 |= (h2[h] > 0.f) ? (1u << h) : 0u;
    }
    masks[0] = m1;
    masks[1] = m2;
  }
}

// HT > 0: fixed shape (fully unrolled); HT == 0: run-time H and F.
template <int HT, int FT, bool REC = false>
__device__ __forceinline__ void mlp_eval(const float x6[6], const float* __restrict__ freq,
                                         const float* __restrict__ att, int F, int H, const MlpPtrs& m, int p,
                                         float out[4], uint32_t* masks = nullptr) {
  if constexpr (HT > 0) mlp_fixed<HT, FT, REC>(x6, freq, att, m, p, out, masks);
  else mlp_generic<REC>(x6, freq, att, F, H, m, p, out, masks);
}

}  // namespace mlpsp
