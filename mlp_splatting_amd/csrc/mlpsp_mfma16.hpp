// Matrix-core (v_mfma_f32_32x32x16, bf16 or fp16 operands, f32 accumulation) evaluation of the per-primitive
// 72->32->32->4 MLP for one wavefront = 64 pixels = two column blocks of 32, shared by the forward render
// (mlpsp_render_mfma.hip) and the training-records forward (mlpsp_records_mfma.hip).
//
// The GEMMs are computed TRANSPOSED: D[hidden][pixel] = W[hidden][k] * X[k][pixel], i.e. the weights are the
// A operand and the pixels are the B/N dimension.  With the 32x32x16 register layout
//     A: lane l holds row  l%32, k = 8*(l/32) + 0..7        B: lane l holds column l%32, same k
//     D: lane l holds column l%32, rows 8*(r/4) + 4*(l/32) + r%4 for r = 0..15
// a lane's D registers of one layer ARE a valid B operand of the next layer (same pixel column, 8 k-slots
// per K-step) provided the next layer's weight columns are stored in that register order.  Weights are
// therefore repacked (pack kernel in mlpsp_render_mfma.hip) into A-fragment order with the k-permutation
// folded in, and the chain layer1 -> ReLU -> layer2 -> ReLU -> layer3 needs no LDS, no barrier and no
// cross-lane traffic until the very end (the four-row output layer runs on 4x4x4 products whose two halves are
// joined by one half-wave swap per output, layer3_small).  Staging a primitive's weights is 7 coalesced 1 KiB loads
// straight into VGPRs (plus two small ones for the four output rows).
//
// Layer-1 k-slots: lane group g = l/32 owns frequencies 3g..3g+2 of every input component, so both groups
// evaluate 18 (sin, cos) pairs per pixel block and each pair lands in one 32-bit operand word.  sin/cos use
// the native v_sin_f32/v_cos_f32 (argument in revolutions); their error (~1e-6) is far below the operand
// rounding applied next.  The 9 words of the ray direction do not depend on the primitive: the caller
// computes them once per pixel (encode_direction_words) and parks them in LDS in operand form.
#pragma once
#include "../../include/mlpsp.h"
#include "mlpsp_device.hpp"

namespace mlpsp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// packed per-primitive block (bytes).  The biases of the two hidden layers travel as operands: b = hi + lo with
// hi = round(b) and lo = round(b - hi) in the operand type (17 significant bits for bf16, 22 for fp16), multiplied
// by a constant (1, 1) operand word and summed in f32 by the MFMA itself.  Layer 1 has spare k-slots for that
// (72 of 80 used), and for the bias of layer 2 as well: its word sits in the last of them, where layer 1 multiplies
// it by zero, and layer 2 gets a third K-step that multiplies the same A operand (the last K-step of W1) by an
// operand that is (1, 1) in that slot and zero elsewhere.  No bias is loaded as a 16-register C operand any more
// (such loads cost the vector-memory pipe as much as the weights themselves), nor as a word of its own.
constexpr int kOffW1 = 0;       // 5 K-steps x 64 lanes x 16 B; words 18, 19 of lane group 0 = (b1 hi, b1 lo), (b2 hi, b2 lo)
constexpr int kOffW2 = 5120;    // 2 K-steps x 64 lanes x 16 B
constexpr int kOffB2 = 7168;    // 256 B, zero (reserved)
constexpr int kOffW3 = 7424;    // 2 K-steps x 2 lane groups x 4 rows x 16 B
constexpr int kOffB3 = 7680;    // 4 f32
constexpr int kOffFlag = 7696;  // int32: 1 if any rounded weight or bias is non-finite
constexpr int kPackStride = MLPSP_MFMA_PACK_BYTES;
static_assert(kPackStride >= kOffFlag + 4 && kPackStride % 128 == 0, "pack stride");

template <typename T> struct Ops;
template <> struct Ops<__bf16> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    bf16x2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(unsigned, v);
  }
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma4(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(i16x4, a), __builtin_bit_cast(i16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float round_trip(float a) { return (float)(__bf16)a; }
  static constexpr unsigned kOneWord = 0x3f803f80u;   // (1, 1)
  static constexpr float kMax = 3.38953139e38f;
  // bf16 has the exponent range of f32: a hidden pre-activation is out of range only if it is (within one
  // rounding step of) +-inf.  Rounded to +inf it survives the ReLU and turns the next layer's sums into
  // +-inf or NaN, down to the outputs, whose finiteness every hit checks; rounded to -inf the ReLU removes
  // it, as it does in exact arithmetic.  The per-layer range check is therefore not needed for this type.
  static constexpr bool kCheckHidden = false;
};
template <> struct Ops<_Float16> {
  using vec8 = f16x8;
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    f16x2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(unsigned, v);
  }
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma4(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float round_trip(float a) { return (float)(_Float16)a; }
  static constexpr unsigned kOneWord = 0x3c003c00u;   // (1, 1)
  static constexpr float kMax = 65504.0f;
  static constexpr bool kCheckHidden = true;   // a finite f32 pre-activation above 65504 must be reported
};

// row of the 32x32 accumulator tile held by D register r of lane group g (fixed by the instruction)
__host__ __device__ constexpr int d_row(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }
// Hidden unit assigned to that row.  Which unit sits in which row is free as long as the pack kernel uses
// one assignment for a layer's output rows, its bias and the next layer's weight columns.  This one makes
// the ReLU masks of the training records cheap: a lane's packed operand word (s, d) holds registers
// r = 8s + 2d (low half) and r + 1 (high half), i.e. units 4s + d + 8g and 16 + 4s + d + 8g, so "half is
// non-zero" shifted left by 4s + d lands on the unit's bit of the 32-bit mask (relu_mask_bits below).
__host__ __device__ constexpr int hidden_unit(int r, int g) { return 16 * (r & 1) + (r >> 1) + 8 * g; }
// ... and the unit held by accumulator row m (the A operand row a lane m%32 loads weights for)
__host__ __device__ constexpr int hidden_unit_of_row(int m) { return hidden_unit(4 * (m >> 3) + (m & 3), (m >> 2) & 1); }

// True if some pre-activation is +-inf or exceeds the operand type's range.  A NaN cannot appear here
// on its own: the operands are finite (weights are checked when packed, phases when encoded), so a
// non-finite accumulator is an overflow, which shows as +-inf -- and the max chain sees infinities.
// ReLU of two packed 16-bit floats in one instruction: as signed 16-bit integers every negative float
// (and -0) is below zero and every non-negative one keeps its bits, for bf16 and fp16 alike; rounding
// commutes with ReLU, so rounding first gives the same operand.
// The instruction itself is left to the compiler, not written as inline assembly: the output layer's 4x4x4 products
// may write another register group than the one they accumulate from, and the compiler keeps the next writer of
// the old group one wait state away from such a product only if it can see that the writer is a vector
// instruction.  The empty statement only hides where x comes from; otherwise the conversion that produced x is
// split into two conversions and a byte permute to fit the integer maximum.
__device__ __forceinline__ unsigned relu_packed(unsigned x) {
  typedef short i16x2 __attribute__((ext_vector_type(2)));
  asm("" : "+v"(x));
  const i16x2 zero = {0, 0};
  return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(i16x2, x), zero));
}
__device__ __forceinline__ float max3_abs(float a, float b, float c) {
  float y;
  asm("v_max3_f32 %0, |%1|, |%2|, |%3|" : "=v"(y) : "v"(a), "v"(b), "v"(c));
  return y;
}
// The first read of the accumulator tile is a plain C++ operation, not inline assembly: the compiler
// inserts the wait states a matrix-core result needs before its first reader only for instructions it
// can see, and everything below depends on that first read.
// (The running maximum is updated in place: an inline-assembly instruction that writes a register of its own
// could be given one that a 4x4x4 product issued just before still reads as its addend.)
template <typename T>
__device__ __forceinline__ bool out_of_range_in(const f32x16& v) {
  float m = __builtin_fabsf(v[0]);
#pragma unroll
  for (int r = 1; r < 15; r += 2) asm("v_max3_f32 %0, |%0|, |%1|, |%2|" : "+v"(m) : "v"(v[r]), "v"(v[r + 1]));
  asm("v_max3_f32 %0, |%0|, |%1|, |%1|" : "+v"(m) : "v"(v[15]));
  return !(m <= Ops<T>::kMax);
}


// Operand words of the ray direction for both column blocks, [block][.][lane]; one wavefront per workgroup
// writes and reads its own copy, so no barrier is needed.
struct DirWords {
  u32x4 q[2][2][64];
  unsigned w8[2][64];
};

// kf[j] = freq * att / (2 pi) of frequency 3g + j: the phase scale, in revolutions per unit input, of the
// three frequencies this lane's group evaluates.
__device__ __forceinline__ void phase_scales(const float* __restrict__ freq, const float* __restrict__ att, int g,
                                             float kf[3]) {
  constexpr float kInvTwoPi = 0.159154943f;
#pragma unroll
  for (int j = 0; j < 3; ++j) kf[j] = (freq[3 * g + j] * att[3 * g + j]) * kInvTwoPi;
}

// sin and cos of the position half of the encoding from a table (forward render, bf16 operands).
//
// Every instruction this kernel issues costs its full issue time -- a transcendental twice and a half that of an
// ordinary vector instruction -- and the 18 (sin, cos) pairs of a hit step were a sixth of it.  A table of
// kSinCosEntries operand words (sin, cos of entry / kSinCosEntries revolutions, already rounded and packed) in the
// workgroup's LDS replaces, per pair, two transcendentals and the pack by one mask and one LDS read: the phase
// x k is formed in units of a quarter table entry by the multiply-add that used to be the multiply,
//     y = fma(x, k * 4 * kSinCosEntries, 1.5 * 2^23 + 2),
// whose low mantissa bits ARE the rounded integer (the constant puts y where floats are spaced one apart), so that
// bits(y) & (4 * kSinCosEntries - 4) is the byte offset of the nearest entry.  The angle is off by at most half an
// entry, pi / 2048 = 1.5e-3 rad: 0.8 of what rounding sin and cos to bf16 costs anyway (fp16 operands, which round
// eight times finer, keep the instructions).  Valid while |x k| < 512 revolutions; the caller checks the inputs.
#ifndef MLPSP_SINCOS_ENTRIES
#define MLPSP_SINCOS_ENTRIES 2048
#endif
constexpr int kSinCosEntries = MLPSP_SINCOS_ENTRIES;
constexpr float kSinCosMagic = 12582912.0f + 2.0f;
constexpr float kSinCosRange = 500.0f;          // revolutions (the multiply-add is exact to an entry below 512)
struct SinCosTable {
  unsigned w[kSinCosEntries];
};
// Filled by the whole workgroup (any size); the caller puts a barrier behind it.
template <typename T>
__device__ __forceinline__ void fill_sincos_table(SinCosTable& t) {
  for (int e = threadIdx.x; e < kSinCosEntries; e += blockDim.x) {
    const float rev = (float)e * (1.0f / (float)kSinCosEntries);
    t.w[e] = Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev));
  }
}
__device__ __forceinline__ unsigned sincos_word(const SinCosTable& t, float x, float k_scaled) {
  const unsigned off = __float_as_uint(fmaf(x, k_scaled, kSinCosMagic)) & (4u * kSinCosEntries - 4u);
  return *reinterpret_cast<const unsigned*>(reinterpret_cast<const unsigned char*>(t.w) + off);
}

template <typename T>
__device__ __forceinline__ void encode_direction_words(float rdx, float rdy, float rdz, const float kf[3], int l,
                                                       DirWords& s) {
  const int g = l >> 5;
  // the pixel this lane shares an MFMA column with: lane l and lane l^32 both hold column l%32
  const float prdx = __shfl_xor(rdx, 32), prdy = __shfl_xor(rdy, 32), prdz = __shfl_xor(rdz, 32);
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const bool own = (b == g);
    const float xd[3] = {own ? rdx : prdx, own ? rdy : prdy, own ? rdz : prdz};
    unsigned wd[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) {
      const float rev = xd[t / 3] * kf[t % 3];
      wd[t] = Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev));
    }
    s.q[b][0][l] = u32x4{wd[0], wd[1], wd[2], wd[3]};
    s.q[b][1][l] = u32x4{wd[4], wd[5], wd[6], wd[7]};
    s.w8[b][l] = wd[8];
  }
}

// Bits 4s+d and 16+4s+d of a lane's partial ReLU mask from the rectified operand word (s, d): a half that is
// not zero is an active unit (the rounded activation the next layer really multiplies).
__device__ __forceinline__ unsigned relu_mask_bits(unsigned rectified, int shift) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  const u16x2 one = {1, 1};
  const u16x2 nz = __builtin_elementwise_min(__builtin_bit_cast(u16x2, rectified), one);
  return __builtin_bit_cast(unsigned, nz) << shift;
}

// (hi, lo) operand word of a bias: hi + lo reproduces b to twice the operand type's precision.
template <typename T>
__device__ __forceinline__ unsigned bias_word(float b) {
  const float hi = Ops<T>::round_trip(b);
  return Ops<T>::pack2(hi, b - hi);
}

// Both halves of the wavefront exchange a value in one instruction: returns {[x lanes 0..31 | x lanes 0..31],
// [x lanes 32..63 | x lanes 32..63]}, i.e. for column block b the value of pixel 32 b + l % 32 in every lane.
struct HalfPair {
  float blk0, blk1;
};
// (The two results are copied into scalars before they are reinterpreted: __builtin_bit_cast applied to an
// element expression of the returned vector reads element 0 whatever the index.)
__device__ __forceinline__ HalfPair both_halves(float x) {
  const unsigned u = __float_as_uint(x);
  // (the swap rewrites both of its operands: given the same value twice the compiler copies it twice; given a
  // second name for it, once)
  unsigned twin = u;
  asm("" : "+v"(twin));
  const auto r = __builtin_amdgcn_permlane32_swap(u, twin, false, false);
  const unsigned lo = r[0], hi = r[1];
  return HalfPair{__uint_as_float(lo), __uint_as_float(hi)};
}

// [a lanes 0..31 + a lanes 32..63 | b lanes 0..31 + b lanes 32..63]
__device__ __forceinline__ float sum_of_halves(float a, float b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  const unsigned lo = r[0], hi = r[1];
  return __uint_as_float(lo) + __uint_as_float(hi);
}

// The output layer has four rows: as a 32x32x16 product 28 of its 32 accumulator rows would be zero.  It runs on
// v_mfma_f32_4x4x4 (sixteen independent 4x4x4 products, one per group of four lanes, 8 clocks) instead: in the
// group of lane l, lane l supplies A row l % 4 = output row l % 4 and B column l % 4 = its own pixel column, four
// k-slots each, and receives the four sums of its own column.  The k-slots a lane can supply are the hidden units
// its accumulator registers hold, so lanes l and l ^ 32 each get one half of the column's sums (added by
// sum_of_halves); a packed row of eight weights (16 bytes, registers 8s .. 8s+7 of lane group g) is two such steps.
template <typename T>
__device__ __forceinline__ f32x4 layer3_small(u32x4 a, u32x4 b, f32x4 c) {
  c = Ops<T>::mfma4(u32x2{a[0], a[1]}, u32x2{b[0], b[1]}, c);
  return Ops<T>::mfma4(u32x2{a[2], a[3]}, u32x2{b[2], b[3]}, c);
}

// The MLP of primitive block `blk` for the pixels of `mask` (ballot of the lanes that hit).  dx, dy, dz: this
// lane's own hit offset (inputs 3..5; lanes that did not hit pass anything finite).  o[k] = output k of THIS
// lane's pixel, output bias included.
// CHECK: report pre-activations outside the operand type's range.  MASKS: also return the pixel's two
// 32-bit ReLU masks (bit u = hidden unit u active) in mk.  Returns true if a stored weight was flagged
// non-finite when packed or (CHECK) a pre-activation of a hit pixel is out of range.
// Vector-memory instructions per call: 7 (W1, W2) + 1 (b2 words) + 2 (W3); the output bias and the flag are
// wave-uniform scalar loads.
// LUT: the position words come from the workgroup's sin/cos table; kf then holds the phase scales times
// 4 kSinCosEntries.
template <typename T, bool CHECK, bool MASKS, bool LUT = false>
__device__ __forceinline__ bool mlp_wave_mfma16(const unsigned char* __restrict__ blk, unsigned long long mask, int l,
                                                float dx, float dy, float dz, const float kf[3], const DirWords& dir,
                                                float o[4], unsigned mk[2], const SinCosTable* table = nullptr) {
  const int g = l >> 5;
  bool bad = false;
  // Addresses of the weight loads: wave-uniform base in scalar registers + zero-extended 32-bit lane offset +
  // immediate, the form the global loads take as they are, so that no address is computed per lane and hit.  The
  // compiler picks that form only if it sees the zero extension next to the load; the lane index is therefore made
  // opaque here, once per call (otherwise the extended offsets are hoisted out of the primitive loop as 64-bit
  // registers and added to the base per lane).  Everything beyond the first 4 KiB of the block is addressed from a
  // second scalar base: the immediates end at 4095.
  int ll = l;
  unsigned row16 = (unsigned)(g * 4 + (l & 3)) * 16u, upper = 4096u;
  asm volatile("" : "+v"(ll), "+v"(row16), "+s"(upper));
  const unsigned lane16 = (unsigned)ll * 16u;
  const unsigned char* hi = blk + upper;
  // ---- stage the primitive's weights: MFMA A fragments, straight from global memory
  u32x4 a1[5], a2[2], a3[2];
#pragma unroll
  for (int s = 0; s < 5; ++s) a1[s] = *reinterpret_cast<const u32x4*>((s < 4 ? blk : hi - 4096) + kOffW1 + s * 1024 + lane16);
#pragma unroll
  for (int s = 0; s < 2; ++s) a2[s] = *reinterpret_cast<const u32x4*>(hi + (kOffW2 - 4096) + s * 1024 + lane16);
#pragma unroll
  // output layer: lane l supplies output row l % 4 for the hidden units its lane group holds (layer3_small)
  for (int s = 0; s < 2; ++s) a3[s] = *reinterpret_cast<const u32x4*>(hi + (kOffW3 - 4096) + s * 128 + row16);
  const f32x4 b3v = *reinterpret_cast<const f32x4*>(blk + kOffB3);
  const int wflag = *reinterpret_cast<const int32_t*>(blk + kOffFlag);
  bad |= (wflag != 0);
  // the constant operand word that multiplies the (hi, lo) bias words: k-slots of lane group 0 only
  const unsigned one_word = g ? 0u : Ops<T>::kOneWord;

  // ---- inputs 3..5 of both column blocks
  const HalfPair hx = both_halves(dx), hy = both_halves(dy), hz = both_halves(dz);
  float o_blk[2][4];
  unsigned m_blk[2][2] = {{0u, 0u}, {0u, 0u}};
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const unsigned half_mask = (unsigned)(mask >> (32 * b));
    if (half_mask != 0u) {   // wave-uniform: skip a 32-pixel block nobody hits
      const float xin[3] = {b ? hx.blk1 : hx.blk0, b ? hy.blk1 : hy.blk0, b ? hz.blk1 : hz.blk0};
      const bool col_active = (half_mask >> (l & 31)) & 1u;
      // layer 1: 18 (sin, cos) words per lane + the bias word, 5 K-steps; words 0..8 come from LDS.  (The lane
      // index is made opaque so that the loads stay here and are not hoisted out of the primitive loop into
      // registers.)
      const u32x4 dq0 = dir.q[b][0][ll], dq1 = dir.q[b][1][ll];
      const unsigned d8 = dir.w8[b][ll];
      f32x16 d1 = zero16;
#pragma unroll
      for (int s = 0; s < 5; ++s) {
        u32x4 bw;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int t = 4 * s + d;
          if (t < 4) {
            bw[d] = dq0[d];
          } else if (t < 8) {
            bw[d] = dq1[d];
          } else if (t == 8) {
            bw[d] = d8;
          } else if (t < 18) {
            if constexpr (LUT) {
              bw[d] = sincos_word(*table, xin[t / 3 - 3], kf[t % 3]);
            } else {
              const float rev = xin[t / 3 - 3] * kf[t % 3];
              bw[d] = Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev));
            }
          } else if (t == 18) {
            bw[d] = one_word;
          } else {
            bw[d] = 0u;
          }
        }
        d1 = Ops<T>::mfma(a1[s], bw, d1);
      }
      if constexpr (CHECK) bad |= col_active && out_of_range_in<T>(d1);
      // layer 2: the bias K-step first (its operands are ready), then the D registers of layer 1, rectified and
      // rounded, as the B operand
      // (its B operand is constant, three zero words and the (1, 1) word: the compiler keeps it in four registers
      // across the primitive loop, which there is room for)
      const unsigned z0 = 0u, z1 = 0u, z2 = 0u;
      f32x16 d2 = Ops<T>::mfma(a1[4], u32x4{z0, z1, z2, one_word}, zero16);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        u32x4 bw;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          bw[d] = relu_packed(Ops<T>::pack2(d1[8 * s + 2 * d], d1[8 * s + 2 * d + 1]));
          if constexpr (MASKS) m_blk[b][0] |= relu_mask_bits(bw[d], 4 * s + d);
        }
        d2 = Ops<T>::mfma(a2[s], bw, d2);
      }
      if constexpr (CHECK) bad |= col_active && out_of_range_in<T>(d2);
      // output layer: this lane's half of the four sums of its column (layer3_small)
      f32x4 d3 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        u32x4 bw;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          bw[d] = relu_packed(Ops<T>::pack2(d2[8 * s + 2 * d], d2[8 * s + 2 * d + 1]));
          if constexpr (MASKS) m_blk[b][1] |= relu_mask_bits(bw[d], 4 * s + d);
        }
        d3 = layer3_small<T>(a3[s], bw, d3);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) o_blk[b][k] = d3[k];
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) o_blk[b][k] = 0.f;
    }
  }
  // pixel l < 32 belongs to block 0, pixel l >= 32 to block 1: both lane groups' halves of its sums
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = sum_of_halves(o_blk[0][k], o_blk[1][k]) + b3v[k];
  if constexpr (MASKS) {
    // lane group g holds the units 8g..8g+7 and 16+8g..16+8g+7 of its column: shift into place, merge the
    // two groups, and take the block this lane's pixel belongs to (block g)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const unsigned mine0 = m_blk[0][j] << (8 * g), mine1 = m_blk[1][j] << (8 * g);
      const unsigned full0 = mine0 | (unsigned)__shfl_xor((int)mine0, 32);
      const unsigned full1 = mine1 | (unsigned)__shfl_xor((int)mine1, 32);
      mk[j] = g ? full1 : full0;
    }
  }
  return bad;
}

// The same evaluation with the two column blocks advanced together, for a wavefront whose hit mask has pixels in
// both halves.  A wavefront's MLP is otherwise one dependent chain (K-step after K-step of a layer, the layer's
// sixteen registers rectified and packed, the next layer, ...), and with four wavefronts per SIMD there is often
// nothing else to issue while an MFMA or its first reader waits.  Here every MFMA of block 0 is followed by the
// independent MFMA of block 1, and the operand preparation of one block sits behind the MFMA of the other.
// No ReLU masks (render only).
template <typename T, bool CHECK, bool LUT = false>
__device__ __forceinline__ bool mlp_pair_mfma16(const unsigned char* __restrict__ blk, unsigned long long mask, int l,
                                                float dx, float dy, float dz, const float kf[3], const DirWords& dir,
                                                float o[4], const SinCosTable* table = nullptr) {
  const int g = l >> 5;
  bool bad = false;
  // Addresses of the weight loads: wave-uniform base in scalar registers + zero-extended 32-bit lane offset +
  // immediate, the form the global loads take as they are, so that no address is computed per lane and hit.  The
  // compiler picks that form only if it sees the zero extension next to the load; the lane index is therefore made
  // opaque here, once per call (otherwise the extended offsets are hoisted out of the primitive loop as 64-bit
  // registers and added to the base per lane).  Everything beyond the first 4 KiB of the block is addressed from a
  // second scalar base: the immediates end at 4095.
  int ll = l;
  unsigned row16 = (unsigned)(g * 4 + (l & 3)) * 16u, upper = 4096u;
  asm volatile("" : "+v"(ll), "+v"(row16), "+s"(upper));
  const unsigned lane16 = (unsigned)ll * 16u;
  const unsigned char* hi = blk + upper;
  u32x4 a1[5], a2[2], a3[2];
#pragma unroll
  for (int s = 0; s < 5; ++s) a1[s] = *reinterpret_cast<const u32x4*>((s < 4 ? blk : hi - 4096) + kOffW1 + s * 1024 + lane16);
#pragma unroll
  for (int s = 0; s < 2; ++s) a2[s] = *reinterpret_cast<const u32x4*>(hi + (kOffW2 - 4096) + s * 1024 + lane16);
#pragma unroll
  for (int s = 0; s < 2; ++s) a3[s] = *reinterpret_cast<const u32x4*>(hi + (kOffW3 - 4096) + s * 128 + row16);
  const f32x4 b3v = *reinterpret_cast<const f32x4*>(blk + kOffB3);
  const int wflag = *reinterpret_cast<const int32_t*>(blk + kOffFlag);
  bad |= (wflag != 0);
  const unsigned one_word = g ? 0u : Ops<T>::kOneWord;
  const HalfPair hx = both_halves(dx), hy = both_halves(dy), hz = both_halves(dz);
  const float xin[2][3] = {{hx.blk0, hy.blk0, hz.blk0}, {hx.blk1, hy.blk1, hz.blk1}};
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16 d1[2] = {zero16, zero16};
  // The wavefront asks for issue priority while it walks its MFMA chains (the other wavefronts of the SIMD are
  // mostly in vector work, which also issues beside an MFMA): 0.7 % off the kernel, measured against priority 0
  // on one device; raising it earlier, over the weight loads, or for the walk instead, gains nothing.
  __builtin_amdgcn_s_setprio(2);
#pragma unroll
  for (int s = 0; s < 5; ++s) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      u32x4 bw;
      if (s == 0) {
        bw = dir.q[b][0][ll];
      } else if (s == 1) {
        bw = dir.q[b][1][ll];
      } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int t = 4 * s + d;
          if (t == 8) {
            bw[d] = dir.w8[b][ll];
          } else if (t < 18) {
            if constexpr (LUT) {
              bw[d] = sincos_word(*table, xin[b][t / 3 - 3], kf[t % 3]);
            } else {
              const float rev = xin[b][t / 3 - 3] * kf[t % 3];
              bw[d] = Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev));
            }
          } else if (t == 18) {
            bw[d] = one_word;
          } else {
            bw[d] = 0u;
          }
        }
      }
      d1[b] = Ops<T>::mfma(a1[s], bw, d1[b]);
    }
  }
  if constexpr (CHECK) {
    bad |= ((mask >> (l & 31)) & 1ull) && out_of_range_in<T>(d1[0]);
    bad |= ((mask >> (32 + (l & 31))) & 1ull) && out_of_range_in<T>(d1[1]);
  }
  const unsigned z0 = 0u, z1 = 0u, z2 = 0u;
  // the bias tile of layer 2 (every column the same) is computed once and is the addend of both blocks' first K-step
  const f32x16 bias2 = Ops<T>::mfma(a1[4], u32x4{z0, z1, z2, one_word}, zero16);
  f32x16 d2[2] = {bias2, bias2};
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      u32x4 bw;
#pragma unroll
      for (int d = 0; d < 4; ++d) bw[d] = relu_packed(Ops<T>::pack2(d1[b][8 * s + 2 * d], d1[b][8 * s + 2 * d + 1]));
      d2[b] = Ops<T>::mfma(a2[s], bw, d2[b]);
    }
  }
  if constexpr (CHECK) {
    bad |= ((mask >> (l & 31)) & 1ull) && out_of_range_in<T>(d2[0]);
    bad |= ((mask >> (32 + (l & 31))) & 1ull) && out_of_range_in<T>(d2[1]);
  }
  f32x4 d3[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      u32x4 bw;
#pragma unroll
      for (int d = 0; d < 4; ++d) bw[d] = relu_packed(Ops<T>::pack2(d2[b][8 * s + 2 * d], d2[b][8 * s + 2 * d + 1]));
      d3[b] = layer3_small<T>(a3[s], bw, d3[b]);
    }
  }
  __builtin_amdgcn_s_setprio(0);
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = sum_of_halves(d3[0][k], d3[1][k]) + b3v[k];
  return bad;
}

}  // namespace mlpsp
