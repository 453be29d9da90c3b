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
// Every intermediate lives in LDS in the layout(s) its consumers need -- row-major [row][k] as an A operand,
// [column][k] as a B operand -- so each MFMA fragment is one aligned LDS read of 16 bytes (16-bit types) or
// one word (f32).  Rows are padded (8 elements / 1 word) to spread the banks.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"

namespace mlpsp {

typedef float vf32x16 __attribute__((ext_vector_type(16)));
typedef unsigned vu32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 vbf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 vf16x8 __attribute__((ext_vector_type(8)));

constexpr int kGradFloats = 3524;   // W1 2304 | b1 32 | W2 1024 | b2 32 | W3 128 | b3 4 (primitive_gemm.py:160-166)

template <typename T> struct Vjp;
template <> struct Vjp<float> {
  static constexpr int KS = 2, KV = 1, PAD = 1;   // k per MFMA, k per lane, row padding (elements)
  using Frag = float;
  static __device__ __forceinline__ Frag load(const float* p) { return *p; }
  static __device__ __forceinline__ vf32x16 mfma(Frag a, Frag b, vf32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Vjp<_Float16> {
  static constexpr int KS = 16, KV = 8, PAD = 8;
  using Frag = vu32x4;
  static __device__ __forceinline__ Frag load(const _Float16* p) { return *reinterpret_cast<const vu32x4*>(p); }
  static __device__ __forceinline__ vf32x16 mfma(Frag a, Frag b, vf32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(vf16x8, a), __builtin_bit_cast(vf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float round(float v) { return (float)(_Float16)v; }
};
template <> struct Vjp<__bf16> {
  static constexpr int KS = 16, KV = 8, PAD = 8;
  using Frag = vu32x4;
  static __device__ __forceinline__ Frag load(const __bf16* p) { return *reinterpret_cast<const vu32x4*>(p); }
  static __device__ __forceinline__ vf32x16 mfma(Frag a, Frag b, vf32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(vbf16x8, a), __builtin_bit_cast(vbf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float round(float v) { return (float)(__bf16)v; }
};

// K rounded up to whole MFMA steps
template <typename T> constexpr int kpad(int k) { return (k + Vjp<T>::KS - 1) / Vjp<T>::KS * Vjp<T>::KS; }

// The LDS tiles of one wavefront.  LD_x = row stride in elements.
template <typename T> struct VjpTiles {
  static constexpr int P = Vjp<T>::PAD;
  static constexpr int K1 = kpad<T>(72), K3 = kpad<T>(4);
  static constexpr int LD1 = K1 + P, LD32 = 32 + P, LD3 = K3 + P;
  T w1[32 * LD1];      // [hid][k]        B operand of the layer-1 forward product
  T w2[32 * LD32];     // [hid2][hid]     B operand of the layer-2 forward product
  T w2t[32 * LD32];    // [hid][hid2]     B operand of D1 = D2 W2
  T w3t[32 * LD3];     // [hid2][out]     B operand of D2 = D3 W3
  T enc[32 * LD1];     // [rec][k]        A operand of layer 1
  T enct[96 * LD32];   // [k][rec]        B operand of gW1 (rows 72..95 stay zero)
  T h1[32 * LD32];     // [rec][hid]      A operand of layer 2
  T h1t[32 * LD32];    // [hid][rec]      B operand of gW2
  T h2t[32 * LD32];    // [hid2][rec]     B operand of gW3
  T d3[32 * LD3];      // [rec][out]      A operand of D2 = D3 W3
  T d3t[32 * LD32];    // [out][rec]      A operand of gW3 (rows 4..31 stay zero)
  T d2[32 * LD32];     // [rec][hid2]     A operand of D1 = D2 W2
  T d2t[32 * LD32];    // [hid2][rec]     A operand of gW2
  T d1t[32 * LD32];    // [hid][rec]      A operand of gW1
  int32_t mask[2][32];
};

// acc += A B with A = a[32 rows][K] and B given as bt[32 columns][K] (both with k contiguous).
template <typename T>
__device__ __forceinline__ vf32x16 mma(const T* a, int lda, const T* bt, int ldb, int K, vf32x16 acc, int lane) {
  constexpr int KS = Vjp<T>::KS, KV = Vjp<T>::KV;
  const int m = lane & 31, g = lane >> 5;
  for (int k = 0; k < K; k += KS)
    acc = Vjp<T>::mfma(Vjp<T>::load(a + m * lda + k + KV * g), Vjp<T>::load(bt + m * ldb + k + KV * g), acc);
  return acc;
}

// Accumulator tile -> LDS, as [row][col] and/or [col][row].  Lane (n, g) holds column n, rows 8q + 4g + r.
template <typename T>
__device__ __forceinline__ void store_tile(const vf32x16& v, T* rowmajor, int ld_r, T* colmajor, int ld_c, int lane) {
  const int n = lane & 31, g = lane >> 5;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = 8 * (i >> 2) + 4 * g + (i & 3);
    if (rowmajor) rowmajor[row * ld_r + n] = (T)v[i];
    if (colmajor) colmajor[n * ld_c + row] = (T)v[i];
  }
}

template <typename T>
__global__ __launch_bounds__(64) void grouped_vjp_kernel(
    const float* __restrict__ x6, const float* __restrict__ grad4, const int32_t* __restrict__ masks,
    const long long* __restrict__ offsets, const long long* __restrict__ group_prim,
    const long long* __restrict__ group_start, const float* __restrict__ freq, const float* __restrict__ att,
    const float* __restrict__ W1, const float* __restrict__ b1, const float* __restrict__ W2,
    const float* __restrict__ b2, const float* __restrict__ W3, float scale, int segment,
    float* __restrict__ partial) {
  using TL = VjpTiles<T>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  TL& t = *reinterpret_cast<TL*>(smem);
  const int lane = threadIdx.x, n = lane & 31, g = lane >> 5;
  const long long group = blockIdx.x;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;

  // ---- zero the tiles (padding columns and the never-written rows must be zero), stage the weights
  {
    unsigned* z = reinterpret_cast<unsigned*>(smem);
    for (int i = lane; i < (int)(sizeof(TL) / 4); i += 64) z[i] = 0u;
  }
  __syncthreads();
  for (int i = lane; i < 32 * 72; i += 64) t.w1[(i / 72) * TL::LD1 + i % 72] = (T)W1[p * 2304 + i];
  for (int i = lane; i < 32 * 32; i += 64) {
    const T w = (T)W2[p * 1024 + i];
    t.w2[(i >> 5) * TL::LD32 + (i & 31)] = w;
    t.w2t[(i & 31) * TL::LD32 + (i >> 5)] = w;
  }
  for (int i = lane; i < 4 * 32; i += 64) t.w3t[(i & 31) * TL::LD3 + (i >> 5)] = (T)W3[p * 128 + i];
  const float bias1 = b1[p * 32 + n], bias2 = b2[p * 32 + n];   // a lane's accumulator column is hidden unit n
  __syncthreads();

  vf32x16 gw1[3], gw2, gw3;
#pragma unroll
  for (int i = 0; i < 16; ++i) gw1[0][i] = gw1[1][i] = gw1[2][i] = gw2[i] = gw3[i] = 0.f;
  float gb1 = 0.f, gb2 = 0.f, gb3 = 0.f;
  const vf32x16 zero = gw2;

  for (long long base = begin; base < end; base += 32) {
    // ---- inputs of this block: lane (n, g) encodes record base + n, pairs 18g .. 18g+17; adjoints; masks
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
        const T ts = live ? (T)s : (T)0.f, tc = live ? (T)co : (T)0.f;
        t.enc[n * TL::LD1 + j] = ts;
        t.enc[n * TL::LD1 + 36 + j] = tc;
        t.enct[j * TL::LD32 + n] = ts;
        t.enct[(36 + j) * TL::LD32 + n] = tc;
      }
    }
    if (g == 0) {
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        const T d = live ? (T)(grad4[rec * 4 + o] * scale) : (T)0.f;
        t.d3[n * TL::LD3 + o] = d;
        t.d3t[o * TL::LD32 + n] = d;
      }
    } else if (masks) {
      t.mask[0][n] = live ? masks[rec * 2] : 0;
      t.mask[1][n] = live ? masks[rec * 2 + 1] : 0;
    }
    __syncthreads();

    // ---- forward: H1, H2 (accumulator column = hidden unit n, rows = records)
    vf32x16 a1 = mma<T>(t.enc, TL::LD1, t.w1, TL::LD1, TL::K1, zero, lane);
    unsigned act1 = 0u, act2 = 0u;   // bit i: the unit is active for the record of accumulator register i
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * g + (i & 3);
      const float h = fmaxf(a1[i] + bias1, 0.f);
      a1[i] = h;
      act1 |= (masks ? ((unsigned)t.mask[0][row] >> n) & 1u : (h > 0.f ? 1u : 0u)) << i;
    }
    store_tile<T>(a1, t.h1, TL::LD32, t.h1t, TL::LD32, lane);
    __syncthreads();
    vf32x16 a2 = mma<T>(t.h1, TL::LD32, t.w2, TL::LD32, 32, zero, lane);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * g + (i & 3);
      const float h = fmaxf(a2[i] + bias2, 0.f);
      a2[i] = h;
      act2 |= (masks ? ((unsigned)t.mask[1][row] >> n) & 1u : (h > 0.f ? 1u : 0u)) << i;
    }
    store_tile<T>(a2, (T*)nullptr, 0, t.h2t, TL::LD32, lane);

    // ---- backward: D2 = (D3 W3) * act2, D1 = (D2 W2) * act1; bias gradients from the rounded adjoints
    vf32x16 dd2 = mma<T>(t.d3, TL::LD3, t.w3t, TL::LD3, TL::K3, zero, lane);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dd2[i] = ((act2 >> i) & 1u) ? dd2[i] : 0.f;
      gb2 += Vjp<T>::round(dd2[i]);
    }
    store_tile<T>(dd2, t.d2, TL::LD32, t.d2t, TL::LD32, lane);
    __syncthreads();
    vf32x16 dd1 = mma<T>(t.d2, TL::LD32, t.w2t, TL::LD32, 32, zero, lane);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dd1[i] = ((act1 >> i) & 1u) ? dd1[i] : 0.f;
      gb1 += Vjp<T>::round(dd1[i]);
    }
    store_tile<T>(dd1, (T*)nullptr, 0, t.d1t, TL::LD32, lane);
    // layer-3 bias: lane o < 4 sums the rounded adjoints of output o over the block's records
    if (lane < 4) {
      for (int r = 0; r < 32; ++r) gb3 += (float)t.d3t[lane * TL::LD32 + r];
    }
    __syncthreads();

    // ---- weight gradients: contraction over the block's 32 records
#pragma unroll
    for (int c = 0; c < 3; ++c)
      gw1[c] = mma<T>(t.d1t, TL::LD32, t.enct + c * 32 * TL::LD32, TL::LD32, 32, gw1[c], lane);
    gw2 = mma<T>(t.d2t, TL::LD32, t.h1t, TL::LD32, 32, gw2, lane);
    gw3 = mma<T>(t.d3t, TL::LD32, t.h2t, TL::LD32, 32, gw3, lane);
    __syncthreads();
  }

  // ---- partial[group]: accumulator column n, rows 8q + 4g + r
  float* __restrict__ out = partial + group * kGradFloats;
  const float inv = 1.f / scale;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = 8 * (i >> 2) + 4 * g + (i & 3);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int k = 32 * c + n;
      if (k < 72) out[row * 72 + k] = gw1[c][i] * inv;
    }
    out[2336 + row * 32 + n] = gw2[i] * inv;
    if (row < 4) out[3392 + row * 32 + n] = gw3[i] * inv;
  }
  // bias gradients: the two lane groups hold complementary rows of the same column
  gb1 += __shfl_xor(gb1, 32);
  gb2 += __shfl_xor(gb2, 32);
  if (g == 0) {
    out[2304 + n] = gb1 * inv;
    out[3360 + n] = gb2 * inv;
  }
  if (lane < 4) out[3520 + lane] = gb3 * inv;
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

// One thread per (primitive, gradient element): sum over the primitive's segments; flag non-finite sums.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial,
                                                              const long long* __restrict__ group_offsets,
                                                              float* __restrict__ out, int32_t* __restrict__ nonfinite) {
  const long long p = blockIdx.x;
  const int k = blockIdx.y * 256 + threadIdx.x;
  const long long start = group_offsets[p], end = group_offsets[p + 1];
  bool bad = false;
  if (k < kGradFloats) {
    float total = 0.f;
    for (long long grp = start; grp < end; ++grp) total += partial[grp * kGradFloats + k];
    out[p * kGradFloats + k] = total;
    bad = !(__builtin_fabsf(total) <= 3.4028235e38f);
  }
  if (__ballot(bad) != 0ull && (threadIdx.x & 63) == 0) atomicOr(nonfinite, 1);
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
    const size_t lds = sizeof(VjpTiles<T>);                                                                        \
    MLPSP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_vjp_kernel<T>),                       \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                      \
    hipLaunchKernelGGL((grouped_vjp_kernel<T>), grid, block, lds, s, x6_dev, grad4_dev, relu_masks_dev,            \
                       (const long long*)csr_offsets_dev, (const long long*)group_primitives_dev,                  \
                       (const long long*)group_starts_dev, freq_dev, att_dev, W1, b1, W2, b2, W3, scale, segment,  \
                       partial_dev);                                                                               \
  } while (0)
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

MLPSP_API int mlpsp_reduce_partials(const float* partial_dev, const int64_t* group_offsets_dev, int num_primitives,
                                    float* out_dev, int32_t* nonfinite_dev, mlpsp_stream_t stream) {
  if (num_primitives < 0) return MLPSP_E_ARGUMENT;
  if (!nonfinite_dev) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(nonfinite_dev, 0, sizeof(int32_t), s));
  if (num_primitives == 0) return MLPSP_OK;
  if (!group_offsets_dev || !out_dev) return MLPSP_E_ARGUMENT;
  // (partial_dev may be null only if no primitive has a segment; the kernel then reads nothing)
  const dim3 grid((unsigned)num_primitives, (kGradFloats + 255) / 256), block(256);
  hipLaunchKernelGGL(reduce_partials_kernel, grid, block, 0, s, partial_dev, (const long long*)group_offsets_dev,
                     out_dev, nonfinite_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
