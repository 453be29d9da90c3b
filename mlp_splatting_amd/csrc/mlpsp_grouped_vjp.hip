// libmlpsp_hip: weight gradients of the per-primitive 72->32->32->4 MLP over a primitive-major CSR of hit
// records (counterpart of the reference's Triton kernels _grouped_vjp and _reduce_partials,
// scannet/primitive_gemm.py:101-183).
//
// One wavefront owns one segment (at most `segment` consecutive records of one primitive) and walks it in
// blocks of 32 records.  Per block it re-computes the forward pass (encoding, two hidden layers), pushes the
// output adjoints back through the layers and accumulates the three weight gradients, all as 32x32 MFMA
// tiles with f32 accumulation over the whole segment:
//     H1 = relu(ENC W1^T + b1)      H2 = relu(H1 W2^T + b2)
//     D2 = (D3 W3) * act2           D1 = (D2 W2) * act1
//     gW1 += D1^T ENC     gW2 += D2^T H1     gW3 += D3^T H2     gb_l += column sums of D_l
// Operand type T: float (v_mfma_f32_32x32x2_f32, an exact IEEE f32 fma chain: the reference's "ieee" path),
// _Float16 or __bf16 (v_mfma_f32_32x32x16).  As in the reference, operands are rounded to T, the adjoint d3 is
// scaled by `scale` before rounding and the result divided by it, and the bias gradients sum the ROUNDED
// adjoints so that biases and matrices see the same values (:168-171).  act_l comes from the saved ReLU masks
// if given, else from the recomputed pre-activations (:148-155).
//
// The 16-bit kernels keep every tile in registers (below); the f32 kernel stages its tiles in LDS (further below).
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mfma16.hpp"
#include "mlpsp_segment_reduce.hpp"

namespace mlpsp {

typedef float vf32x16 __attribute__((ext_vector_type(16)));

constexpr int kGradFloats = 3524;   // W1 2304 | b1 32 | W2 1024 | b2 32 | W3 128 | b3 4 (primitive_gemm.py:160-166)

// ---------------------------------------------------------------------------------------------
// The 16-bit paths (fp16 / bf16 operands, v_mfma_f32_32x32x16, f32 accumulation): everything in registers.
//
// An MFMA D = A B takes from lane (m, g) row m of A and column m of B, eight k-slots each (k = 8 g + 0..7
// of the K-step), and returns to lane (n, g) column n of D, rows d_row(i, g) = 8 (i/4) + 4 g + i%4 in
// register i.  Two consequences carry the whole kernel:
//  (1) Swapping the operands transposes the result: with X = the block's 32 records (one per lane, k-slots =
//      its inputs) and W = a weight matrix (one output unit per lane), mfma(W, X) puts a RECORD in every lane
//      and the units in its registers ("record-major" tile), mfma(X, W) a UNIT in every lane and the records
//      d_row(i, g) in its registers ("unit-major").  A record-major tile, rectified, rounded and packed in
//      pairs, is the X operand of the next layer; a unit-major tile packed the same way is an operand whose
//      k-slots are RECORDS -- which is what the weight gradients contract over.  Since both operands of a
//      weight-gradient product come from unit-major tiles, their k-slots name the same records, and nothing has
//      to be transposed through LDS: each forward/backward product is simply issued in both orientations.
//  (2) A tile that no product yields in the needed orientation (the encoding, the output adjoints) is
//      transposed by the matrix core itself: mfma(X, I) with a 0/1 selection operand I returns X unit-major,
//      exactly (one non-zero term per sum).
// Per block of 32 records: 32 MFMAs (34 without saved masks) against 20 for a formulation that transposes
// through LDS, and no LDS traffic except the 64 mask words: 11.3 -> 2.8 ms for 38.6 M records, with one
// wavefront per SIMD (342 registers; capped at 256 the compiler spills 84 and the kernel takes 4.5 ms).
//
// k-slot order of the encoding (both the X operand of layer 1 and W1's operand): lane group g owns input
// components 3g..3g+2; its slot q = 8 s + j of K-step s (q < 36) is pair t = q / 2 = 6 c + f (component
// 3g + c, frequency f), sin for even q, cos for odd.  Slots q = 36..39 are padding; slot q = 36 of group 0
// (k = 68) carries the constant 1, so that the layer-1 bias gradient falls out of the W1 product as one more
// column.  sin/cos use the native v_sin/v_cos in revolutions: their error (~1e-6) is far below the operand
// rounding, as in the forward kernels of this precision.
// ---------------------------------------------------------------------------------------------
typedef unsigned short vu16x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Unpack;
template <> struct Unpack<__bf16> {
  static __device__ __forceinline__ float lo(unsigned w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(unsigned w) { return __uint_as_float(w & 0xFFFF0000u); }
};
template <> struct Unpack<_Float16> {
  static __device__ __forceinline__ float lo(unsigned w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
  static __device__ __forceinline__ float hi(unsigned w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
};

// 0xFFFF in every half of `rectified` that is not zero (an active unit), 0 in the others
__device__ __forceinline__ unsigned active_halves(unsigned rectified) {
  const vu16x2 one = {1, 1}, all = {0xFFFF, 0xFFFF};
  return __builtin_bit_cast(unsigned, (vu16x2)(__builtin_elementwise_min(__builtin_bit_cast(vu16x2, rectified), one) * all));
}

struct Pack8 {
  u32x4 s[2];   // the two K-steps of a 32-deep contraction
};

template <typename T>
__device__ __forceinline__ Pack8 pack_tile(const vf32x16& v) {
  Pack8 r;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) r.s[s][d] = Ops<T>::pack2(v[8 * s + 2 * d], v[8 * s + 2 * d + 1]);
  return r;
}
__device__ __forceinline__ Pack8 relu_tile(Pack8 r) {
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) r.s[s][d] = relu_packed(r.s[s][d]);
  return r;
}
__device__ __forceinline__ Pack8 and_tile(Pack8 r, const Pack8& m) {
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) r.s[s][d] &= m.s[s][d];
  return r;
}
__device__ __forceinline__ Pack8 active_tile(const Pack8& h) {
  Pack8 r;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) r.s[s][d] = active_halves(h.s[s][d]);
  return r;
}
// AND-masks of a unit-major tile from saved mask words: w[i] = the mask word of the record in register i,
// bit = this lane's unit
__device__ __forceinline__ Pack8 mask_tile_unit_major(const int32_t w[16], int bit) {
  Pack8 r;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int i = 8 * s + 2 * d;
      const unsigned lo = (unsigned)__builtin_amdgcn_sbfe(w[i], bit, 1), hi = (unsigned)__builtin_amdgcn_sbfe(w[i + 1], bit, 1);
      r.s[s][d] = (lo & 0xFFFFu) | (hi << 16);
    }
  return r;
}
// ... and of a record-major tile: `word` = the mask word of this lane's record, register i is unit d_row(i, g)
__device__ __forceinline__ Pack8 mask_tile_record_major(int32_t word, int g) {
  const int shifted = word >> (4 * g);
  Pack8 r;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int i = 8 * s + 2 * d, u = 8 * (i / 4) + (i % 4);      // d_row(i, 0); i is even, so i + 1 is unit u + 1
      const unsigned lo = (unsigned)__builtin_amdgcn_sbfe(shifted, u, 1), hi = (unsigned)__builtin_amdgcn_sbfe(shifted, u + 1, 1);
      r.s[s][d] = (lo & 0xFFFFu) | (hi << 16);
    }
  return r;
}
template <typename T>
__device__ __forceinline__ float sum_tile(const Pack8& r) {
  float t = 0.f;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int d = 0; d < 4; ++d) t += Unpack<T>::lo(r.s[s][d]) + Unpack<T>::hi(r.s[s][d]);
  return t;
}
template <typename T>
__device__ __forceinline__ vf32x16 mma2(const Pack8& a, const Pack8& b, vf32x16 acc) {
  acc = Ops<T>::mfma(a.s[0], b.s[0], acc);
  return Ops<T>::mfma(a.s[1], b.s[1], acc);
}
__device__ __forceinline__ vf32x16 splat16(float v) {
  vf32x16 r;
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = v;
  return r;
}

template <typename T, bool SAVED>
__global__ __launch_bounds__(64) void grouped_vjp16_kernel(
    const float* __restrict__ x6, const float* __restrict__ grad4, const int32_t* __restrict__ masks,
    const long long* __restrict__ offsets, const long long* __restrict__ group_prim,
    const long long* __restrict__ group_start, const float* __restrict__ freq, const float* __restrict__ att,
    const float* __restrict__ W1, const float* __restrict__ b1, const float* __restrict__ W2,
    const float* __restrict__ b2, const float* __restrict__ W3, float scale, int segment,
    float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) int32_t s_mask[2][32];
  const int lane = threadIdx.x, n = lane & 31, g = lane >> 5;
  const long long group = blockIdx.x;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;

  // ---- the primitive's weights as operands, one unit (n) per lane
  u32x4 w1op[5];
  {
    const float* __restrict__ row = W1 + p * 2304 + n * 72 + 18 * g;
    float ws[18], wc[18];
#pragma unroll
    for (int t = 0; t < 18; t += 2) {
      const float2 a = *reinterpret_cast<const float2*>(row + t), c = *reinterpret_cast<const float2*>(row + 36 + t);
      ws[t] = a.x;
      ws[t + 1] = a.y;
      wc[t] = c.x;
      wc[t + 1] = c.y;
    }
#pragma unroll
    for (int s = 0; s < 5; ++s)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int t = 4 * s + d;
        w1op[s][d] = t < 18 ? Ops<T>::pack2(ws[t], wc[t]) : 0u;
      }
  }
  Pack8 w2op, w2top;     // W2[n][u] and W2[u][n] over the units u = d_row(8 s + j, g) of this lane's k-slots
  {
    const float* __restrict__ row = W2 + p * 1024 + n * 32;
    const float* __restrict__ col = W2 + p * 1024 + n;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const float4 lo = *reinterpret_cast<const float4*>(row + 16 * s + 4 * g);
      const float4 hi = *reinterpret_cast<const float4*>(row + 16 * s + 8 + 4 * g);
      w2op.s[s] = u32x4{Ops<T>::pack2(lo.x, lo.y), Ops<T>::pack2(lo.z, lo.w), Ops<T>::pack2(hi.x, hi.y), Ops<T>::pack2(hi.z, hi.w)};
      float c[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) c[j] = col[(16 * s + 8 * (j / 4) + 4 * g + j % 4) * 32];
      w2top.s[s] = u32x4{Ops<T>::pack2(c[0], c[1]), Ops<T>::pack2(c[2], c[3]), Ops<T>::pack2(c[4], c[5]), Ops<T>::pack2(c[6], c[7])};
    }
  }
  // W3^T: k-slots = the four outputs (group 0, slots 0..3)
  u32x4 w3op = {0u, 0u, 0u, 0u};
  if (g == 0) {
    const float* __restrict__ col = W3 + p * 128 + n;
    w3op[0] = Ops<T>::pack2(col[0], col[32]);
    w3op[1] = Ops<T>::pack2(col[64], col[96]);
  }
  // selection operands: out_sel returns the output adjoints unit-major (column n = output n < 4); k_sel[h]
  // returns K-step 2c + h of the encoding as columns 32c + n
  const unsigned one_lo = Ops<T>::pack2(1.f, 0.f), one_hi = Ops<T>::pack2(0.f, 1.f);
  u32x4 out_sel = {0u, 0u, 0u, 0u};
  if (g == 0 && n < 4) out_sel[n >> 1] = (n & 1) ? one_hi : one_lo;
  u32x4 k_sel[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
  {
    const unsigned v = (n & 1) ? one_hi : one_lo;
    const bool mine = ((n >> 3) & 1) == g;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int d = 0; d < 4; ++d) k_sel[h][d] = (mine && (n >> 4) == h && ((n & 7) >> 1) == d) ? v : 0u;
  }
  const float bias1 = b1[p * 32 + n], bias2 = b2[p * 32 + n];
  float kf[6];
#pragma unroll
  for (int f = 0; f < 6; ++f) kf[f] = (freq[f] * att[f]) * 0.159154943f;

  vf32x16 gw1[3], gw2, gw3;
#pragma unroll
  for (int i = 0; i < 16; ++i) gw1[0][i] = gw1[1][i] = gw1[2][i] = gw2[i] = gw3[i] = 0.f;
  float gb2 = 0.f, gb3[4] = {0.f, 0.f, 0.f, 0.f};
  const vf32x16 zero = gw2;

  for (long long base = begin; base < end; base += 32) {
    const long long rec = base + n;
    const bool live = rec < end;
    // ---- this lane's record: three inputs of its group, the output adjoints, the mask words
    float x[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) x[c] = live ? x6[rec * 6 + 3 * g + c] : 0.f;
    float4 d3 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live && g == 0) d3 = *reinterpret_cast<const float4*>(grad4 + rec * 4);
    int32_t mine_mask = 0;
    if constexpr (SAVED) {
      mine_mask = live ? masks[rec * 2 + g] : 0;      // group 0 fetches layer 1, group 1 layer 2
      s_mask[g][n] = mine_mask;
    }
    // ---- encoding, record-major
    u32x4 enc[5];
#pragma unroll
    for (int s = 0; s < 5; ++s)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int t = 4 * s + d;
        if (t < 18) {
          const float rev = x[t / 6] * kf[t % 6];
          enc[s][d] = live ? Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev)) : 0u;
        } else if (t == 18) {
          enc[s][d] = (live && g == 0) ? one_lo : 0u;      // the constant input (k = 68): bias gradient of layer 1
        } else {
          enc[s][d] = 0u;
        }
      }
    u32x4 d3op = {0u, 0u, 0u, 0u};                        // rounded, scaled output adjoints (group 0)
    d3op[0] = Ops<T>::pack2(d3.x * scale, d3.y * scale);
    d3op[1] = Ops<T>::pack2(d3.z * scale, d3.w * scale);
    gb3[0] += Unpack<T>::lo(d3op[0]);
    gb3[1] += Unpack<T>::hi(d3op[0]);
    gb3[2] += Unpack<T>::lo(d3op[1]);
    gb3[3] += Unpack<T>::hi(d3op[1]);

    // ---- layer 1 in both orientations
    vf32x16 a_rec, a_unit = splat16(bias1);
    {
      // record-major: register i is unit d_row(i, g); its bias comes from global memory (L1-resident)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 v = *reinterpret_cast<const float4*>(b1 + p * 32 + 8 * q + 4 * g);
        a_rec[4 * q] = v.x;
        a_rec[4 * q + 1] = v.y;
        a_rec[4 * q + 2] = v.z;
        a_rec[4 * q + 3] = v.w;
      }
    }
#pragma unroll
    for (int s = 0; s < 5; ++s) {
      a_rec = Ops<T>::mfma(w1op[s], enc[s], a_rec);
      a_unit = Ops<T>::mfma(enc[s], w1op[s], a_unit);
    }
    const Pack8 h1_rec = relu_tile(pack_tile<T>(a_rec));
    const Pack8 h1_unit = relu_tile(pack_tile<T>(a_unit));
    // ---- layer 2: unit-major for the W3 gradient; record-major only to learn which units are active
    const Pack8 h2_unit = relu_tile(pack_tile<T>(mma2<T>(h1_rec, w2op, splat16(bias2))));
    Pack8 act1_unit, act2_unit, act2_rec;
    if constexpr (SAVED) {
      int32_t w[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int4 v = *reinterpret_cast<const int4*>(&s_mask[0][8 * q + 4 * g]);
        w[4 * q] = v.x;
        w[4 * q + 1] = v.y;
        w[4 * q + 2] = v.z;
        w[4 * q + 3] = v.w;
      }
      act1_unit = mask_tile_unit_major(w, n);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int4 v = *reinterpret_cast<const int4*>(&s_mask[1][8 * q + 4 * g]);
        w[4 * q] = v.x;
        w[4 * q + 1] = v.y;
        w[4 * q + 2] = v.z;
        w[4 * q + 3] = v.w;
      }
      act2_unit = mask_tile_unit_major(w, n);
      act2_rec = mask_tile_record_major(s_mask[1][n], g);
    } else {
      vf32x16 a2;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 v = *reinterpret_cast<const float4*>(b2 + p * 32 + 8 * q + 4 * g);
        a2[4 * q] = v.x;
        a2[4 * q + 1] = v.y;
        a2[4 * q + 2] = v.z;
        a2[4 * q + 3] = v.w;
      }
      act1_unit = active_tile(h1_unit);
      act2_unit = active_tile(h2_unit);
      act2_rec = active_tile(relu_tile(pack_tile<T>(mma2<T>(w2op, h1_rec, a2))));
    }
    // ---- backward: D2 in both orientations, D1 unit-major, the output adjoints unit-major
    const Pack8 d2_rec = and_tile(pack_tile<T>(Ops<T>::mfma(w3op, d3op, zero)), act2_rec);
    const Pack8 d2_unit = and_tile(pack_tile<T>(Ops<T>::mfma(d3op, w3op, zero)), act2_unit);
    const Pack8 d1_unit = and_tile(pack_tile<T>(mma2<T>(d2_rec, w2top, zero)), act1_unit);
    const Pack8 d3_unit = pack_tile<T>(Ops<T>::mfma(d3op, out_sel, zero));
    gb2 += sum_tile<T>(d2_unit);
    // ---- weight gradients: contraction over the records in the k-slots of the unit-major tiles
    gw2 = mma2<T>(d2_unit, h1_unit, gw2);
    gw3 = mma2<T>(d3_unit, h2_unit, gw3);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      vf32x16 e = Ops<T>::mfma(enc[2 * c], k_sel[0], zero);
      if (c < 2) e = Ops<T>::mfma(enc[2 * c + 1], k_sel[1], e);
      gw1[c] = mma2<T>(d1_unit, pack_tile<T>(e), gw1[c]);
    }
  }

  // ---- partial[group]: accumulator column n, rows d_row(i, g)
  float* __restrict__ out = partial + group * kGradFloats;
  const float inv = 1.f / scale;
  int feature[3];       // W1 column of encoding slot k = 32 c + n; -1: padding, -2: the constant input
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const int k = 32 * c + n, q = 8 * (k >> 4) + (k & 7), gk = (k >> 3) & 1;
    feature[c] = q < 36 ? (q & 1) * 36 + 18 * gk + (q >> 1) : ((q == 36 && gk == 0) ? -2 : -1);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = 8 * (i >> 2) + 4 * g + (i & 3);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      if (feature[c] >= 0) out[row * 72 + feature[c]] = gw1[c][i] * inv;
      else if (feature[c] == -2) out[2304 + row] = gw1[c][i] * inv;
    }
    out[2336 + row * 32 + n] = gw2[i] * inv;
    if (row < 4) out[3392 + row * 32 + n] = gw3[i] * inv;
  }
  gb2 += __shfl_xor(gb2, 32);
  if (g == 0) out[3360 + n] = gb2 * inv;
#pragma unroll
  for (int o = 0; o < 4; ++o) {
    float v = gb3[o];
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m);
    if (lane == o) out[3520 + o] = v * inv;
  }
}

// ---------------------------------------------------------------------------------------------
// The f32 path.  v_mfma_f32_32x32x2_f32 takes ONE element per lane and operand, so an operand can be read from
// LDS in either orientation and no transposed copies are needed; and the contraction over the block's records
// may run in any order, so the weight-gradient products take their A operand -- an adjoint tile, transposed --
// straight from the accumulator registers that hold it: register i of lane (column c, group g) is row
// rec(i, g) = 8 (i / 4) + 4 g + i % 4, which is used as "record 2 i + g" of the contraction, the B operand
// reading the same record's row.  Tiles in LDS: encoding, both hidden activations, d2 and d3 (row-major,
// [record][column]) and the weights in their own layout: 37 KB per wavefront, four wavefronts per CU.
// ---------------------------------------------------------------------------------------------
struct VjpTilesF32 {
  static constexpr int LD1 = 73, LD32 = 33, LD3 = 5;
  float w1[32 * LD1];    // [hid][k]
  float w2[32 * LD32];   // [hid2][hid]
  float w3[4 * LD32];    // [out][hid2]
  float enc[32 * LD1];   // [rec][k]
  float h1[32 * LD32];   // [rec][hid]
  float h2[32 * LD32];   // [rec][hid2]
  float d2[32 * LD32];   // [rec][hid2]
  float d3[32 * LD3];    // [rec][out]
  int32_t mask[2][32];
};

__device__ __forceinline__ vf32x16 mfma32(float a, float b, vf32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// acc += A B over STEPS MFMAs; element k of the operands at a[k * a_stride], b[k * b_stride] (the caller folds
// the lane's row/column and k-group into the pointers).  Operands are fetched CHUNK steps ahead of the MFMAs
// that use them: written as "load, wait, MFMA" per step the LDS latency is paid once per instruction.
template <int STEPS, int CHUNK>
__device__ __forceinline__ vf32x16 mma_f32(const float* a, int a_stride, const float* b, int b_stride, vf32x16 acc) {
  static_assert(STEPS % CHUNK == 0, "whole chunks");
#pragma unroll
  for (int c0 = 0; c0 < STEPS; c0 += CHUNK) {
    float av[CHUNK], bv[CHUNK];
#pragma unroll
    for (int s = 0; s < CHUNK; ++s) {
      av[s] = a[(c0 + s) * a_stride];
      bv[s] = b[(c0 + s) * b_stride];
    }
#pragma unroll
    for (int s = 0; s < CHUNK; ++s) acc = mfma32(av[s], bv[s], acc);
  }
  return acc;
}

__global__ __launch_bounds__(64) void grouped_vjp_f32_kernel(
    const float* __restrict__ x6, const float* __restrict__ grad4, const int32_t* __restrict__ masks,
    const long long* __restrict__ offsets, const long long* __restrict__ group_prim,
    const long long* __restrict__ group_start, const float* __restrict__ freq, const float* __restrict__ att,
    const float* __restrict__ W1, const float* __restrict__ b1, const float* __restrict__ W2,
    const float* __restrict__ b2, const float* __restrict__ W3, float scale, int segment,
    float* __restrict__ partial) {
  using TL = VjpTilesF32;
  __shared__ TL t;
  const int lane = threadIdx.x, n = lane & 31, g = lane >> 5;
  const long long group = blockIdx.x;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;
  for (int i = lane; i < 32 * 72; i += 64) t.w1[(i / 72) * TL::LD1 + i % 72] = W1[p * 2304 + i];
  for (int i = lane; i < 32 * 32; i += 64) t.w2[(i >> 5) * TL::LD32 + (i & 31)] = W2[p * 1024 + i];
  for (int i = lane; i < 4 * 32; i += 64) t.w3[(i >> 5) * TL::LD32 + (i & 31)] = W3[p * 128 + i];
  const float bias1 = b1[p * 32 + n], bias2 = b2[p * 32 + n];
  __syncthreads();

  vf32x16 gw1[3], gw2, gw3;
#pragma unroll
  for (int i = 0; i < 16; ++i) gw1[0][i] = gw1[1][i] = gw1[2][i] = gw2[i] = gw3[i] = 0.f;
  float gb1 = 0.f, gb2 = 0.f, gb3 = 0.f;
  const vf32x16 zero = gw2;
  const int n2 = n < 8 ? n : 0;    // column of the third 32-wide block of the 72 encoding columns (64 + n2)

  for (long long base = begin; base < end; base += 32) {
    const long long rec = base + n;
    const bool live = rec < end;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const float x = live ? x6[rec * 6 + 3 * g + c] : 0.f;
#pragma unroll
      for (int f = 0; f < 6; ++f) {
        const int j = (3 * g + c) * 6 + f;
        float s, co;
        det_sincos((x * freq[f]) * att[f], s, co);
        t.enc[n * TL::LD1 + j] = live ? s : 0.f;
        t.enc[n * TL::LD1 + 36 + j] = live ? co : 0.f;
      }
    }
    if (g == 0) {
#pragma unroll
      for (int o = 0; o < 4; ++o) t.d3[n * TL::LD3 + o] = live ? grad4[rec * 4 + o] * scale : 0.f;
    } else if (masks) {
      t.mask[0][n] = live ? masks[rec * 2] : 0;
      t.mask[1][n] = live ? masks[rec * 2 + 1] : 0;
    }
    __syncthreads();

    // forward (accumulator column = hidden unit n, register i = record 8 (i/4) + 4 g + i%4)
    vf32x16 a1 = mma_f32<36, 18>(t.enc + n * TL::LD1 + g, 2, t.w1 + n * TL::LD1 + g, 2, zero);
    unsigned act1 = 0u, act2 = 0u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * g + (i & 3);
      const float h = fmaxf(a1[i] + bias1, 0.f);
      t.h1[row * TL::LD32 + n] = h;
      act1 |= (masks ? ((unsigned)t.mask[0][row] >> n) & 1u : (h > 0.f ? 1u : 0u)) << i;
    }
    __syncthreads();
    vf32x16 a2 = mma_f32<16, 16>(t.h1 + n * TL::LD32 + g, 2, t.w2 + n * TL::LD32 + g, 2, zero);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * g + (i & 3);
      const float h = fmaxf(a2[i] + bias2, 0.f);
      t.h2[row * TL::LD32 + n] = h;
      act2 |= (masks ? ((unsigned)t.mask[1][row] >> n) & 1u : (h > 0.f ? 1u : 0u)) << i;
    }
    // backward
    vf32x16 dd2 = mma_f32<2, 2>(t.d3 + n * TL::LD3 + g, 2, t.w3 + g * TL::LD32 + n, 2 * TL::LD32, zero);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * g + (i & 3);
      dd2[i] = ((act2 >> i) & 1u) ? dd2[i] : 0.f;
      gb2 += dd2[i];
      t.d2[row * TL::LD32 + n] = dd2[i];
    }
    if (lane < 4) {
      for (int r = 0; r < 32; ++r) gb3 += t.d3[r * TL::LD3 + lane];
    }
    __syncthreads();
    vf32x16 dd1 = mma_f32<16, 16>(t.d2 + n * TL::LD32 + g, 2, t.w2 + g * TL::LD32 + n, 2 * TL::LD32, zero);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dd1[i] = ((act1 >> i) & 1u) ? dd1[i] : 0.f;
      gb1 += dd1[i];
    }
    // weight gradients: A = the adjoint tile from registers, B = the activation row of the same record
#pragma unroll
    for (int i0 = 0; i0 < 16; i0 += 4) {      // operands of four records ahead of their twenty MFMAs
      float e0[4], e1[4], e2[4], v1[4], v2[4], v3[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u, row = 8 * (i >> 2) + 4 * g + (i & 3);
        e0[u] = t.enc[row * TL::LD1 + n];
        e1[u] = t.enc[row * TL::LD1 + 32 + n];
        e2[u] = t.enc[row * TL::LD1 + 64 + n2];
        v1[u] = t.h1[row * TL::LD32 + n];
        v2[u] = t.h2[row * TL::LD32 + n];
        v3[u] = t.d3[row * TL::LD3 + (n < 4 ? n : 0)];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u;
        gw1[0] = mfma32(dd1[i], e0[u], gw1[0]);
        gw1[1] = mfma32(dd1[i], e1[u], gw1[1]);
        gw1[2] = mfma32(dd1[i], e2[u], gw1[2]);
        gw2 = mfma32(dd2[i], v1[u], gw2);
        gw3 = mfma32(n < 4 ? v3[u] : 0.f, v2[u], gw3);
      }
    }
    __syncthreads();
  }

  float* __restrict__ out = partial + group * kGradFloats;
  const float inv = 1.f / scale;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = 8 * (i >> 2) + 4 * g + (i & 3);
    out[row * 72 + n] = gw1[0][i] * inv;
    out[row * 72 + 32 + n] = gw1[1][i] * inv;
    if (n < 8) out[row * 72 + 64 + n] = gw1[2][i] * inv;
    out[2336 + row * 32 + n] = gw2[i] * inv;
    if (row < 4) out[3392 + row * 32 + n] = gw3[i] * inv;
  }
  gb1 += __shfl_xor(gb1, 32);
  gb2 += __shfl_xor(gb2, 32);
  if (g == 0) {
    out[2304 + n] = gb1 * inv;
    out[3360 + n] = gb2 * inv;
  }
  if (lane < 4) out[3520 + lane] = gb3 * inv;
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_grouped_vjp(const float* x6_dev, const float* grad4_dev, const int32_t* relu_masks_dev,
                                const int64_t* csr_offsets_dev, const int64_t* group_primitives_dev,
                                const int64_t* group_starts_dev, int64_t num_groups, const float* freq_dev,
                                const float* att_dev, const float* W1, const float* b1, const float* W2,
                                const float* b2, const float* W3, int precision, float scale, int segment,
                                float* partial_dev, mlpsp_stream_t stream) {
  if (num_groups < 0 || num_groups > 2147483647LL || segment <= 0 || segment % 32 != 0) return MLPSP_E_ARGUMENT;
  if (precision < 0 || precision > 2 || !(scale > 0.f) || !(scale <= 3.4028235e38f)) return MLPSP_E_ARGUMENT;
  if (num_groups == 0) return MLPSP_OK;
  if (!x6_dev || !grad4_dev || !csr_offsets_dev || !group_primitives_dev || !group_starts_dev || !freq_dev ||
      !att_dev || !W1 || !b1 || !W2 || !b2 || !W3 || !partial_dev)
    return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)num_groups), block(64);
#define MLPSP_VJP_LAUNCH(T)                                                                                        \
  do {                                                                                                             \
    if (relu_masks_dev)                                                                                            \
      hipLaunchKernelGGL((grouped_vjp16_kernel<T, true>), grid, block, 0, s, x6_dev, grad4_dev, relu_masks_dev,    \
                         (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,                \
                         (const long long*)group_starts_dev, freq_dev, att_dev, W1, b1, W2, b2, W3, scale,         \
                         segment, partial_dev);                                                                    \
    else                                                                                                           \
      hipLaunchKernelGGL((grouped_vjp16_kernel<T, false>), grid, block, 0, s, x6_dev, grad4_dev, relu_masks_dev,   \
                         (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,                \
                         (const long long*)group_starts_dev, freq_dev, att_dev, W1, b1, W2, b2, W3, scale,         \
                         segment, partial_dev);                                                                    \
  } while (0)
  if (precision != 0 && ((reinterpret_cast<uintptr_t>(W1) | reinterpret_cast<uintptr_t>(W2) |
                          reinterpret_cast<uintptr_t>(b1) | reinterpret_cast<uintptr_t>(b2) |
                          reinterpret_cast<uintptr_t>(grad4_dev)) & 15) != 0)
    return MLPSP_E_ARGUMENT;      // the 16-bit kernels read weight rows and adjoints with 16-byte loads
  if (precision == 0)
    hipLaunchKernelGGL(grouped_vjp_f32_kernel, grid, block, 0, s, x6_dev, grad4_dev, relu_masks_dev,
                       (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,
                       (const long long*)group_starts_dev, freq_dev, att_dev, W1, b1, W2, b2, W3, scale, segment,
                       partial_dev);
  else if (precision == 1) MLPSP_VJP_LAUNCH(_Float16);
  else MLPSP_VJP_LAUNCH(__bf16);
#undef MLPSP_VJP_LAUNCH
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int64_t mlpsp_segment_reduce_rows(int64_t num_groups) {
  return num_groups < 0 ? -1 : segment_reduce_rows(num_groups);
}

MLPSP_API int mlpsp_reduce_partials(const float* partial_dev, const int64_t* group_primitives_dev,
                                    const int64_t* group_offsets_dev, int64_t num_groups, int num_primitives,
                                    float* out_dev, int32_t* nonfinite_dev, mlpsp_stream_t stream) {
  if (!nonfinite_dev || num_primitives < 0) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(nonfinite_dev, 0, sizeof(int32_t), s));
  ReduceDest dest{};
  dest.packed = out_dev;
  return segment_reduce<false>(partial_dev, group_primitives_dev, group_offsets_dev, num_groups, num_primitives,
                               kGradFloats, dest, nonfinite_dev, s);
}

MLPSP_API int mlpsp_reduce_partials_split(const float* partial_dev, const int64_t* group_primitives_dev,
                                          const int64_t* group_offsets_dev, int64_t num_groups, int num_primitives,
                                          float* gW1_dev, float* gb1_dev, float* gW2_dev, float* gb2_dev, float* gW3_dev,
                                          float* gb3_dev, int32_t* nonfinite_dev, mlpsp_stream_t stream) {
  if (!nonfinite_dev || num_primitives < 0) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(nonfinite_dev, 0, sizeof(int32_t), s));
  ReduceDest dest{};
  float* parts[6] = {gW1_dev, gb1_dev, gW2_dev, gb2_dev, gW3_dev, gb3_dev};
  for (int i = 0; i < 6; ++i) dest.part[i] = parts[i];
  return segment_reduce<true>(partial_dev, group_primitives_dev, group_offsets_dev, num_groups, num_primitives,
                              kGradFloats, dest, nonfinite_dev, s);
}
