// Wave-level f32 evaluation of one primitive's 72->32->32->4 (or 72->16->16->4) MLP for the 64 pixels of a
// wavefront on the matrix cores, bit-identical to the scalar chain of mlp_fixed<32, 6> (mlp_fixed<16, 6>).
//
// v_mfma_f32_32x32x2_f32 computes, per output element, fma(a1, b1, fma(a0, b0, c)) with both steps
// rounded as IEEE f32 fused multiply-adds (no flush of denormals): one instruction is two consecutive links
// of the reference's accumulation chain (np_tile_kernels.cu:2050-2089), so 36 of them walk layer 1 in the
// order sin_j, cos_j and 16 walk layer 2 in the order h = 2i, 2i+1.
//
// Operand layout.  The wavefront's pixels form two column blocks (pixels 0..31 and 32..63), one accumulator
// tile each.  Lane (n = lane % 32, g = lane / 32) of a 32x32 f32 accumulator tile holds column n and rows
// 8q + 4g + r in register 4q + r.  The weight rows are fed in permuted order -- row 8q + 4g + r of the
// A operand is hidden unit 2(4q + r) + g -- so register i of lane (n, g) holds hidden unit 2i + g: exactly
// the B operand (k = g) of the next layer's i-th instruction.  Layer outputs therefore feed the next layer
// from registers, with a ReLU in between and no shuffles.  Layer-1 inputs are computed per lane = pixel and
// moved into operand position by one half-wave swap per sin/cos pair; the same swap brings the 32 layer-2
// outputs of a pixel onto its own lane for the 4-wide output layer, which runs on the vector ALU with
// scalar weight operands.
// With 16 hidden units the same tiles are half filled: A rows 16..31 are zero, accumulator registers 8..15 are
// never read, layer 2 is eight instructions.  The order of every sum is unchanged.
#pragma once
#include "mlpsp_device.hpp"

namespace mlpsp {

typedef float mf32x16 __attribute__((ext_vector_type(16)));
typedef float mf32x4 __attribute__((ext_vector_type(4)));

// Exchanges lanes 32..63 of a with lanes 0..31 of b.
__device__ __forceinline__ void half_swap(float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void half_swap(uint32_t& a, uint32_t& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

// 16 consecutive floats at src + 16 g, as loaded (c[q] = floats 4q .. 4q+3)  ->  element i = src[2i + g]
// (g = lane / 32): eight swaps pair the even entries of the two half-waves.
__device__ __forceinline__ void interleave16(const mf32x4 c4[4], float v[16]) {
  float c[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    c[4 * q + 0] = c4[q][0];
    c[4 * q + 1] = c4[q][1];
    c[4 * q + 2] = c4[q][2];
    c[4 * q + 3] = c4[q][3];
  }
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    half_swap(c[2 * t], c[2 * t + 1]);   // c[2t] = (src[2t], src[2t+1]), c[2t+1] = (src[16+2t], src[17+2t])
    v[t] = c[2 * t];
    v[8 + t] = c[2 * t + 1];
  }
}

// 8 consecutive floats at src + 8 g, as loaded  ->  element i = src[2i + g], i < 8 (the rest of v is left alone).
__device__ __forceinline__ void interleave8(const mf32x4 c4[2], float v[16]) {
  float c[8];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    c[4 * q + 0] = c4[q][0];
    c[4 * q + 1] = c4[q][1];
    c[4 * q + 2] = c4[q][2];
    c[4 * q + 3] = c4[q][3];
  }
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    half_swap(c[2 * t], c[2 * t + 1]);   // c[2t] = (src[2t], src[2t+1]), c[2t+1] = (src[8+2t], src[9+2t])
    v[t] = c[2 * t];
    v[4 + t] = c[2 * t + 1];
  }
}
template <int H>
__device__ __forceinline__ void interleave(const mf32x4 c4[H / 8], float v[16]) {
  if constexpr (H == 32) interleave16(c4, v);
  else interleave8(c4, v);
}

// What one lane loads of a primitive's layers 1 and 2, as the loads deliver it: row `hid` of W1 (its half g) and
// the first bias vector (its half g); the same row of W2 and the second bias vector.  Requesting is separate from
// using, and layer 1 from layer 2: a caller can have the next primitive's layer-1 operands under way while it
// evaluates this one, and layer 2's arrive behind layer 1's instructions anyway.
template <int H>
struct MlpLayer1 {
  mf32x4 a1[9], b1[H / 8];
};
template <int H>
struct MlpLayer2 {
  mf32x4 a2[H / 8], b2[H / 8];
};
// Hidden unit whose weight row lane (m, g) supplies.
__device__ __forceinline__ int mfma32_hidden_row(int m) { return 8 * (m >> 3) + 2 * (m & 3) + ((m >> 2) & 1); }
template <int H>
__device__ __forceinline__ void request_layer1(const float* __restrict__ W1, const float* __restrict__ b1, int p,
                                               MlpLayer1<H>& o) {
  constexpr int IN = 72, HALF = 36;
  const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
  const int hid = mfma32_hidden_row(m);
  const int row = hid < H ? hid : 0;                       // unused rows read row 0 and supply zeros
  const mf32x4* __restrict__ s1 = reinterpret_cast<const mf32x4*>(W1 + (size_t)p * (H * IN) + row * IN + HALF * g);
#pragma unroll
  for (int q = 0; q < 9; ++q) o.a1[q] = s1[q];
  const mf32x4* __restrict__ sb1 = reinterpret_cast<const mf32x4*>(b1 + (size_t)p * H + (H / 2) * g);
#pragma unroll
  for (int q = 0; q < H / 8; ++q) o.b1[q] = sb1[q];
}
template <int H>
__device__ __forceinline__ void request_layer2(const float* __restrict__ W2, const float* __restrict__ b2, int p,
                                               MlpLayer2<H>& o) {
  const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
  const int hid = mfma32_hidden_row(m);
  const int row = hid < H ? hid : 0;
  const mf32x4* __restrict__ s2 = reinterpret_cast<const mf32x4*>(W2 + (size_t)p * (H * H) + row * H + (H / 2) * g);
  const mf32x4* __restrict__ sb2 = reinterpret_cast<const mf32x4*>(b2 + (size_t)p * H + (H / 2) * g);
#pragma unroll
  for (int q = 0; q < H / 8; ++q) {
    o.a2[q] = s2[q];
    o.b2[q] = sb2[q];
  }
}

// max(x, +0): v_max_f32 yields the same bits as x > 0 ? x : 0 for every x (NaN -> 0, -0 -> +0).  Written
// as a builtin, not as inline assembly: the compiler must see the instruction to keep the wait states
// between a matrix-core result and its first reader.
__device__ __forceinline__ float relu_f32(float x) { return __builtin_fmaxf(x, 0.f); }

// The encoding of the ray direction (input components 0..2) does not depend on the primitive: its 18
// sin/cos pairs are computed once per pixel and kept in B-operand position (after the half-wave swap).
struct DirOperands {
  float b0[18], b1[18];
};
__device__ __forceinline__ void encode_direction(float rdx, float rdy, float rdz, const float* __restrict__ freq,
                                                 const float* __restrict__ att, DirOperands& d) {
  const float x3[3] = {rdx, rdy, rdz};
#pragma unroll
  for (int c = 0; c < 3; ++c) {
#pragma unroll
    for (int f = 0; f < 6; ++f) {
      float s, co;
      det_sincos((x3[c] * freq[f]) * att[f], s, co);
      half_swap(s, co);
      d.b0[c * 6 + f] = s;
      d.b1[c * 6 + f] = co;
    }
  }
}

// All 64 lanes must be active.  x6 is the lane's own pixel's input (components 0..2 enter through dir,
// which encode_direction() made from them); out is the lane's own pixel's output.  `w1`, `w2` = the primitive's
// operands as request_layer1() and request_layer2() loaded them.
// REC selects the record kernels' layer-2 rounding (bias added after a chain started at zero); MASKS fills
// masks[0..1] with the ReLU masks of the lane's pixel.
template <bool REC = false, bool MASKS = REC, int HID = 32>
__device__ __forceinline__ void mlp_wave_mfma32_with(const MlpLayer1<HID>& w1, const MlpLayer2<HID>& w2, const float x6[6],
                                                     const float* __restrict__ freq, const float* __restrict__ att,
                                                     const float* __restrict__ W3, const float* __restrict__ b3, int p,
                                                     const DirOperands& dir, float out[4], uint32_t* masks = nullptr) {
  static_assert(HID == 32 || HID == 16, "hidden width of the matrix-core f32 evaluation");
  constexpr int H = HID, R = H / 2;   // R: accumulator registers in use (hidden units 2i + g)
  const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
  const bool row_used = mfma32_hidden_row(m) < H;          // (always, with 32 hidden units)

  // A operands: lane (m, g) supplies row hid, k = g of every instruction.
  float a1[36];
#pragma unroll
  for (int q = 0; q < 9; ++q) {
    a1[4 * q + 0] = row_used ? w1.a1[q][0] : 0.f;
    a1[4 * q + 1] = row_used ? w1.a1[q][1] : 0.f;
    a1[4 * q + 2] = row_used ? w1.a1[q][2] : 0.f;
    a1[4 * q + 3] = row_used ? w1.a1[q][3] : 0.f;
  }
  float a2[16] = {}, bias1[16] = {}, bias2[16] = {};
  interleave<H>(w2.a2, a2);
  interleave<H>(w1.b1, bias1);
  interleave<H>(w2.b2, bias2);
  if constexpr (H != 32) {
#pragma unroll
    for (int i = 0; i < R; ++i) a2[i] = row_used ? a2[i] : 0.f;
  }

  mf32x16 d0, d1;
#pragma unroll
  for (int i = 0; i < 16; ++i) d0[i] = d1[i] = (i < R) ? bias1[i] : 0.f;
#pragma unroll
  for (int j = 0; j < 18; ++j) {
    d0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[j], dir.b0[j], d0, 0, 0, 0);
    d1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[j], dir.b1[j], d1, 0, 0, 0);
  }
#pragma unroll
  for (int c = 3; c < 6; ++c) {
#pragma unroll
    for (int f = 0; f < 6; ++f) {
      float s, co;
      det_sincos((x6[c] * freq[f]) * att[f], s, co);
      half_swap(s, co);   // s: (sin, cos) of pixels 0..31, co: (sin, cos) of pixels 32..63
      d0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[c * 6 + f], s, d0, 0, 0, 0);
      d1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[c * 6 + f], co, d1, 0, 0, 0);
    }
  }

  mf32x16 e0, e1;
#pragma unroll
  for (int i = 0; i < 16; ++i) e0[i] = e1[i] = (REC || i >= R) ? 0.f : bias2[i];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    e0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[i], relu_f32(d0[i]), e0, 0, 0, 0);
    e1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[i], relu_f32(d1[i]), e1, 0, 0, 0);
  }
  if constexpr (REC) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      e0[i] = bias2[i] + e0[i];
      e1[i] = bias2[i] + e1[i];
    }
  }

  // Output layer on the lane's own pixel: register i of the two blocks, swapped, is (h2[2i], h2[2i+1]).
  const float* __restrict__ w3 = W3 + (size_t)p * (4 * H);
  const float* __restrict__ bb3 = b3 + (size_t)p * 4;
  float acc[4] = {bb3[0], bb3[1], bb3[2], bb3[3]};
  uint32_t m2 = 0u;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    float even = relu_f32(e0[i]), odd = relu_f32(e1[i]);
    half_swap(even, odd);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      acc[k] = fmaf(w3[k * H + 2 * i], even, acc[k]);
      acc[k] = fmaf(w3[k * H + 2 * i + 1], odd, acc[k]);
    }
    if constexpr (MASKS) m2 |= (even > 0.f ? (1u << (2 * i)) : 0u) | (odd > 0.f ? (2u << (2 * i)) : 0u);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) out[k] = acc[k];
  if constexpr (MASKS) {
    uint32_t lo = 0u, hi = 0u;   // bits 2i + g of blocks 0 and 1, as held by this lane
#pragma unroll
    for (int i = 0; i < R; ++i) {
      lo |= d0[i] > 0.f ? (1u << (2 * i + g)) : 0u;
      hi |= d1[i] > 0.f ? (1u << (2 * i + g)) : 0u;
    }
    half_swap(lo, hi);
    masks[0] = lo | hi;
    masks[1] = m2;
  }
}

// One column block: the 32 pixels of HALF a wavefront's usual share, every pixel on two lanes (n, g = 0 / 1) that
// hold the same pixel state.  Half the matrix instructions of mlp_wave_mfma32_with() per wavefront -- what a launch
// too small to fill the chip wants, whose time is the time of one wavefront's chain.  Lane (n, g) supplies k = g of
// every B operand itself (the sine for g = 0, the cosine for g = 1: no swap), the layer-2 results of a pixel are
// split over its two lanes as before and one swap per pair brings both to both.  dir[j]: the direction half of the
// encoding in that form (encode_direction_half).  Same chain, same bits.
__device__ __forceinline__ void encode_direction_half(float rdx, float rdy, float rdz, const float* __restrict__ freq,
                                                      const float* __restrict__ att, float dir[18]) {
  const int g = (threadIdx.x & 63) >> 5;
  const float x3[3] = {rdx, rdy, rdz};
#pragma unroll
  for (int c = 0; c < 3; ++c) {
#pragma unroll
    for (int f = 0; f < 6; ++f) {
      float s, co;
      det_sincos((x3[c] * freq[f]) * att[f], s, co);
      dir[c * 6 + f] = g ? co : s;
    }
  }
}
template <int HID>
__device__ __forceinline__ void mlp_half_mfma32_with(const MlpLayer1<HID>& w1, const MlpLayer2<HID>& w2,
                                                     const float x6[6], const float* __restrict__ freq,
                                                     const float* __restrict__ att, const float* __restrict__ W3,
                                                     const float* __restrict__ b3, int p, const float dir[18],
                                                     float out[4]) {
  static_assert(HID == 32 || HID == 16, "hidden width of the matrix-core f32 evaluation");
  constexpr int H = HID, R = H / 2;
  const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
  const bool row_used = mfma32_hidden_row(m) < H;
  float a1[36];
#pragma unroll
  for (int q = 0; q < 9; ++q) {
    a1[4 * q + 0] = row_used ? w1.a1[q][0] : 0.f;
    a1[4 * q + 1] = row_used ? w1.a1[q][1] : 0.f;
    a1[4 * q + 2] = row_used ? w1.a1[q][2] : 0.f;
    a1[4 * q + 3] = row_used ? w1.a1[q][3] : 0.f;
  }
  float a2[16] = {}, bias1[16] = {}, bias2[16] = {};
  interleave<H>(w2.a2, a2);
  interleave<H>(w1.b1, bias1);
  interleave<H>(w2.b2, bias2);
  if constexpr (H != 32) {
#pragma unroll
    for (int i = 0; i < R; ++i) a2[i] = row_used ? a2[i] : 0.f;
  }
  mf32x16 d;
#pragma unroll
  for (int i = 0; i < 16; ++i) d[i] = (i < R) ? bias1[i] : 0.f;
#pragma unroll
  for (int j = 0; j < 18; ++j) d = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[j], dir[j], d, 0, 0, 0);
#pragma unroll
  for (int c = 3; c < 6; ++c) {
#pragma unroll
    for (int f = 0; f < 6; ++f) {
      float s, co;
      det_sincos((x6[c] * freq[f]) * att[f], s, co);
      d = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[c * 6 + f], g ? co : s, d, 0, 0, 0);
    }
  }
  mf32x16 e;
#pragma unroll
  for (int i = 0; i < 16; ++i) e[i] = (i >= R) ? 0.f : bias2[i];
#pragma unroll
  for (int i = 0; i < R; ++i) e = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[i], relu_f32(d[i]), e, 0, 0, 0);

  const float* __restrict__ w3 = W3 + (size_t)p * (4 * H);
  const float* __restrict__ bb3 = b3 + (size_t)p * 4;
  float acc[4] = {bb3[0], bb3[1], bb3[2], bb3[3]};
#pragma unroll
  for (int i = 0; i < R; ++i) {
    // register i of lane (n, g) is hidden unit 2i + g of pixel n: after the swap `even` holds the g = 0 lane's
    // value and `odd` the g = 1 lane's, on both lanes
    float even = relu_f32(e[i]), odd = even;
    half_swap(even, odd);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      acc[k] = fmaf(w3[k * H + 2 * i], even, acc[k]);
      acc[k] = fmaf(w3[k * H + 2 * i + 1], odd, acc[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) out[k] = acc[k];
}

// The same with the operands requested here.
template <bool REC = false, bool MASKS = REC, int HID = 32>
__device__ __forceinline__ void mlp_wave_mfma32(const float x6[6], const float* __restrict__ freq,
                                                const float* __restrict__ att, const float* __restrict__ W1,
                                                const float* __restrict__ b1, const float* __restrict__ W2,
                                                const float* __restrict__ b2, const float* __restrict__ W3,
                                                const float* __restrict__ b3, int p, const DirOperands& dir,
                                                float out[4], uint32_t* masks = nullptr) {
  MlpLayer1<HID> w1;
  MlpLayer2<HID> w2;
  request_layer1<HID>(W1, b1, p, w1);
  request_layer2<HID>(W2, b2, p, w2);
  mlp_wave_mfma32_with<REC, MASKS, HID>(w1, w2, x6, freq, att, W3, b3, p, dir, out, masks);
}

}  // namespace mlpsp
