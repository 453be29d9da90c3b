// libmlpsp_hip: tile-centre-order forward render with the 72->32->32->4 MLP on the matrix cores.
//
// Counterpart of the reference's tensor-core kernel (scannet/cuda/rgb_wmma.cuh:75-223): geometry,
// activations and compositing stay f32; encoded inputs, weights and hidden activations are rounded
// to bf16 (or fp16) and multiplied with v_mfma_f32_32x32x16 with f32 accumulation.
//
// Shape of the work.  One wavefront = one 8x8 tile = 64 pixels = two MFMA column blocks of 32.
// The GEMMs are computed TRANSPOSED: D[hidden][pixel] = W[hidden][k] * X[k][pixel], i.e. the weights
// are the A operand and the pixels are the B/N dimension.  With the 32x32x16 register layout
//     A: lane l holds row  l%32, k = 8*(l/32) + 0..7        B: lane l holds column l%32, same k
//     D: lane l holds column l%32, rows 8*(r/4) + 4*(l/32) + r%4 for r = 0..15
// a lane's D registers of one layer ARE a valid B operand of the next layer (same pixel column, 8
// k-slots per K-step) provided the next layer's weight columns are stored in that register order.
// Weights are therefore repacked once per scene (pack kernel below) into MFMA A-fragment order with
// the k-permutation folded in, and the chain layer1 -> ReLU -> layer2 -> ReLU -> layer3 needs no LDS,
// no barrier and no cross-lane traffic at all.  Staging a primitive's weights is 9 coalesced 1 KiB
// loads straight into VGPRs.
//
// Layer-1 k-slots: lane group g = l/32 owns frequencies 3g..3g+2 of every input component, so both
// groups evaluate 18 (sin, cos) pairs per pixel block and each pair lands in one 32-bit operand word.
// sin/cos use the native v_sin_f32/v_cos_f32 (argument in revolutions); their error (~1e-6) is far
// below the bf16 rounding applied next.  (Measured alternatives that did not pay on gfx950: a 4096-entry
// LDS sin/cos table -- same kernel time, 2x the image error; persistent wavefronts with a tile work
// queue -- 6 % slower than one wavefront per tile.)
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"

namespace mlpsp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// packed per-primitive block (bytes)
constexpr int kOffW1 = 0;       // 5 K-steps x 64 lanes x 16 B
constexpr int kOffW2 = 5120;    // 2 K-steps x 64 lanes x 16 B
constexpr int kOffW3 = 7168;    // 2 K-steps x 2 lane groups x 4 rows x 16 B
constexpr int kOffB1 = 7424;    // 2 lane groups x 16 f32 in D-register order
constexpr int kOffB2 = 7552;
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
  static __device__ __forceinline__ float round_trip(float a) { return (float)(__bf16)a; }
  static constexpr float kMax = 3.38953139e38f;
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
  static __device__ __forceinline__ float round_trip(float a) { return (float)(_Float16)a; }
  static constexpr float kMax = 65504.0f;
};

// hidden-unit index held by D register r of lane group g
__host__ __device__ constexpr int d_row(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }

// ---------------------------------------------------------------------------------------------
// pack: f32 [N,32,72] [N,32] [N,32,32] [N,32] [N,4,32] [N,4]  ->  N blocks of kPackStride bytes
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void pack_mfma_weights_kernel(const float* __restrict__ W1, const float* __restrict__ b1,
                                                               const float* __restrict__ W2, const float* __restrict__ b2,
                                                               const float* __restrict__ W3, const float* __restrict__ b3,
                                                               int N, unsigned char* __restrict__ out) {
  const int p = blockIdx.x;
  if (p >= N) return;
  const int l = threadIdx.x, m = l & 31, g = l >> 5;
  unsigned char* blk = out + (size_t)p * kPackStride;
  const float* w1 = W1 + (size_t)p * 32 * 72 + m * 72;
  const float* w2 = W2 + (size_t)p * 32 * 32 + m * 32;
  bool bad = false;
  auto pk = [&](float a, float b) {
    bad |= !(__builtin_fabsf(Ops<T>::round_trip(a)) <= Ops<T>::kMax) || !(__builtin_fabsf(Ops<T>::round_trip(b)) <= Ops<T>::kMax);
    return Ops<T>::pack2(a, b);
  };
  for (int s = 0; s < 5; ++s) {
    u32x4 v;
    for (int d = 0; d < 4; ++d) {
      const int t = 4 * s + d;
      float ws = 0.f, wc = 0.f;
      if (t < 18) {
        const int j = (t / 3) * 6 + 3 * g + (t % 3);
        ws = w1[j];
        wc = w1[36 + j];
      }
      v[d] = pk(ws, wc);
    }
    *reinterpret_cast<u32x4*>(blk + kOffW1 + s * 1024 + l * 16) = v;
  }
  for (int s = 0; s < 2; ++s) {
    u32x4 v;
    for (int d = 0; d < 4; ++d) v[d] = pk(w2[d_row(8 * s + 2 * d, g)], w2[d_row(8 * s + 2 * d + 1, g)]);
    *reinterpret_cast<u32x4*>(blk + kOffW2 + s * 1024 + l * 16) = v;
  }
  if (l < 16) {
    const int row = l & 3, gg = (l >> 2) & 1, s = l >> 3;
    const float* w3 = W3 + (size_t)p * 4 * 32 + row * 32;
    u32x4 v;
    for (int d = 0; d < 4; ++d) v[d] = pk(w3[d_row(8 * s + 2 * d, gg)], w3[d_row(8 * s + 2 * d + 1, gg)]);
    *reinterpret_cast<u32x4*>(blk + kOffW3 + ((s * 2 + gg) * 4 + row) * 16) = v;
  }
  if (l < 32) {
    const int r = l & 15, gg = l >> 4;
    const float v1 = b1[(size_t)p * 32 + d_row(r, gg)], v2 = b2[(size_t)p * 32 + d_row(r, gg)];
    bad |= !(__builtin_fabsf(v1) <= 3.4028235e38f) || !(__builtin_fabsf(v2) <= 3.4028235e38f);
    reinterpret_cast<float*>(blk + kOffB1)[gg * 16 + r] = v1;
    reinterpret_cast<float*>(blk + kOffB2)[gg * 16 + r] = v2;
  }
  if (l < 4) {
    const float v3 = b3[(size_t)p * 4 + l];
    bad |= !(__builtin_fabsf(v3) <= 3.4028235e38f);
    reinterpret_cast<float*>(blk + kOffB3)[l] = v3;
  }
  const unsigned long long any = __ballot(bad);
  if (l == 0) *reinterpret_cast<int32_t*>(blk + kOffFlag) = any ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------
// render
// ---------------------------------------------------------------------------------------------

// True if some pre-activation is +-inf or exceeds the operand type's range.  A NaN cannot appear here
// on its own: the operands are finite (weights are checked when packed, phases when encoded), so a
// non-finite accumulator is an overflow, which shows as +-inf -- and the max chain sees infinities.
// One-instruction forms.  fmaxf() in C costs two (the compiler first quiets a possible signalling NaN
// with v_max x,x,x), which would double the 64 ReLUs per (tile, primitive).
__device__ __forceinline__ float relu(float x) {
  float y;
  asm("v_max_f32_e32 %0, 0, %1" : "=v"(y) : "v"(x));
  return y;
}
__device__ __forceinline__ float max3_abs(float a, float b, float c) {
  float y;
  asm("v_max3_f32 %0, |%1|, |%2|, |%3|" : "=v"(y) : "v"(a), "v"(b), "v"(c));
  return y;
}
template <typename T>
__device__ __forceinline__ bool out_of_range_in(const f32x16& v) {
  float m = max3_abs(v[0], v[1], v[2]);
#pragma unroll
  for (int r = 3; r < 15; r += 2) m = max3_abs(m, v[r], v[r + 1]);
  m = max3_abs(m, v[15], v[15]);
  return !(m <= Ops<T>::kMax);
}

// f32 activations with the native exp2/log2/rcp instructions (relative error ~1e-6, far below the
// operand rounding of this path).  Same formulas as np_tile_kernels.cu:75-83, 2092-2103.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504f); }
__device__ __forceinline__ float fast_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.0f + fast_exp(-x)); }
__device__ __forceinline__ float fast_softplus(float x) {
  const float e = fast_exp(x);
  const float mid = __builtin_amdgcn_logf(1.0f + e) * 0.693147181f;
  float y = (x < -20.f) ? e : mid;
  y = (x > 20.f) ? x : y;
  return y;
}
__device__ __forceinline__ void fast_blend_step(PixelAcc& a, float o0, float o1, float o2, float o3, float decay) {
  const float sigma = fast_softplus(o3) * decay;
  const float alpha = 1.f - fast_exp(-sigma);
  const float w = a.trans * alpha;
  a.cr = fmaf(w, fast_sigmoid(o0), a.cr);
  a.cg = fmaf(w, fast_sigmoid(o1), a.cg);
  a.cb = fmaf(w, fast_sigmoid(o2), a.cb);
  a.trans = a.trans * (1.f - alpha);
}

template <typename T>
__global__ __launch_bounds__(64) void render_tilecenter_mfma_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, const unsigned char* __restrict__ packed, int N, int W, int H, int ntx,
    int per_xcd, int num_tiles, float thr, float* __restrict__ out_rgb, float* __restrict__ out_alpha,
    int32_t* __restrict__ status, unsigned long long* __restrict__ counters) {
  // XCD-aware work assignment: XCD k (blockIdx.x % 8) walks tiles [k*per_xcd, (k+1)*per_xcd) in
  // row-major order, so neighbouring tiles -- which share most primitives -- run together on one L2.
  const int tile = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (tile >= num_tiles) return;
  const int l = threadIdx.x, g = l >> 5;
  // per-lane phase scales, freq_f * att_f / (2 pi) revolutions per unit input: lane group g evaluates
  // frequencies 3g, 3g+1, 3g+2
  constexpr float kInvTwoPi = 0.159154943f;
  const float kf0 = (freq[3 * g + 0] * att[3 * g + 0]) * kInvTwoPi;
  const float kf1 = (freq[3 * g + 1] * att[3 * g + 1]) * kInvTwoPi;
  const float kf2 = (freq[3 * g + 2] * att[3 * g + 2]) * kInvTwoPi;
  unsigned n_proc = 0, n_proc_hit = 0, n_hits = 0;
  bool bad = false;
  const int tx = tile % ntx, ty = tile / ntx;
  const int x = tx * 8 + (l & 7), y = ty * 8 + (l >> 3);
  const bool valid = (x < W) && (y < H);
  const int pix = valid ? (y * W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f, roy = valid ? rays_o[pix * 3 + 1] : 0.f,
              roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f, rdy = valid ? rays_d[pix * 3 + 1] : 0.f,
              rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  // the pixel this lane shares an MFMA column with: lane l and lane l^32 both hold column l%32
  const float prdx = __shfl_xor(rdx, 32), prdy = __shfl_xor(rdy, 32), prdz = __shfl_xor(rdz, 32);

  const int start = offsets[tile], end = offsets[tile + 1];
  PixelAcc acc = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};

  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool live = valid && (acc.trans >= kTransmittanceFloor);
    const bool hit = live && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    const unsigned long long mask = __ballot(hit);
    ++n_proc;
    if (mask != 0ull) {
      ++n_proc_hit;
      n_hits += __popcll(mask);
      const unsigned char* __restrict__ blk = packed + (size_t)p * kPackStride;
      // ---- stage the primitive's weights: MFMA A fragments, straight from global memory
      u32x4 a1[5], a2[2], a3[2];
#pragma unroll
      for (int s = 0; s < 5; ++s) a1[s] = *reinterpret_cast<const u32x4*>(blk + kOffW1 + s * 1024 + l * 16);
#pragma unroll
      for (int s = 0; s < 2; ++s) a2[s] = *reinterpret_cast<const u32x4*>(blk + kOffW2 + s * 1024 + l * 16);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        a3[s] = u32x4{0u, 0u, 0u, 0u};
        if ((l & 31) < 4) a3[s] = *reinterpret_cast<const u32x4*>(blk + kOffW3 + ((s * 2 + g) * 4 + (l & 3)) * 16);
      }
      const f32x4 b3v = *reinterpret_cast<const f32x4*>(blk + kOffB3);
      const int wflag = *reinterpret_cast<const int32_t*>(blk + kOffFlag);
      bad |= (wflag != 0);
      bad |= hit && !(__builtin_fabsf((h.dx + h.dy) + h.dz) <= 3.4028235e38f);

      // ---- inputs of the column partner
      const float pdx = __shfl_xor(h.dx, 32), pdy = __shfl_xor(h.dy, 32), pdz = __shfl_xor(h.dz, 32);
      float o_blk[2][4];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const unsigned half_mask = (unsigned)(mask >> (32 * b));
        if (half_mask != 0u) {   // wave-uniform: skip a 32-pixel block nobody hits
          const bool own = (b == g);
          const float xin[6] = {own ? rdx : prdx, own ? rdy : prdy, own ? rdz : prdz,
                                own ? h.dx : pdx, own ? h.dy : pdy, own ? h.dz : pdz};
          const bool col_active = (half_mask >> (l & 31)) & 1u;
          // biases are the C operand of each layer's first MFMA; an MFMA overwrites its C registers,
          // so each column block fetches its own copy (L1-resident) instead of copying 32 registers
          f32x16 d1, d2;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x4 v1 = *reinterpret_cast<const f32x4*>(blk + kOffB1 + g * 64 + q * 16);
            const f32x4 v2 = *reinterpret_cast<const f32x4*>(blk + kOffB2 + g * 64 + q * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              d1[4 * q + e] = v1[e];
              d2[4 * q + e] = v2[e];
            }
          }
          // layer 1: 18 (sin, cos) words per lane, 5 K-steps
#pragma unroll
          for (int s = 0; s < 5; ++s) {
            u32x4 bw;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const int t = 4 * s + d;
              if (t < 18) {
                const float kf = (t % 3 == 0) ? kf0 : ((t % 3 == 1) ? kf1 : kf2);
                const float rev = xin[t / 3] * kf;
                bw[d] = Ops<T>::pack2(__builtin_amdgcn_sinf(rev), __builtin_amdgcn_cosf(rev));
              } else {
                bw[d] = 0u;
              }
            }
            d1 = Ops<T>::mfma(a1[s], bw, d1);
          }
          bad |= col_active && out_of_range_in<T>(d1);
          // layer 2: the D registers, rectified and rounded, are the next B operand
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            u32x4 bw;
#pragma unroll
            for (int d = 0; d < 4; ++d)
              bw[d] = Ops<T>::pack2(relu(d1[8 * s + 2 * d]), relu(d1[8 * s + 2 * d + 1]));
            d2 = Ops<T>::mfma(a2[s], bw, d2);
          }
          bad |= col_active && out_of_range_in<T>(d2);
          // layer 3: rows 0..3 of a 32-row product; row k lands in register k of lane group 0
          f32x16 d3 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            u32x4 bw;
#pragma unroll
            for (int d = 0; d < 4; ++d)
              bw[d] = Ops<T>::pack2(relu(d2[8 * s + 2 * d]), relu(d2[8 * s + 2 * d + 1]));
            d3 = Ops<T>::mfma(a3[s], bw, d3);
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) o_blk[b][k] = d3[k];
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k) o_blk[b][k] = 0.f;
        }
      }
      // pixel l < 32 reads block 0 from its own lane; pixel l >= 32 reads block 1 from lane l-32
      float o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float from_partner = __shfl_xor(o_blk[1][k], 32);
        o[k] = (g ? from_partner : o_blk[0][k]) + b3v[k];
      }
      if (hit) {
        bad |= !(__builtin_fabsf(o[0]) <= 3.4028235e38f) || !(__builtin_fabsf(o[1]) <= 3.4028235e38f) ||
               !(__builtin_fabsf(o[2]) <= 3.4028235e38f) || !(__builtin_fabsf(o[3]) <= 3.4028235e38f);
        fast_blend_step(acc, o[0], o[1], o[2], o[3], h.decay);
      }
    }
    if (__ballot(valid && (acc.trans >= kTransmittanceFloor)) == 0ull) break;
  }

  if (valid) {
    out_rgb[pix * 3 + 0] = acc.cr;
    out_rgb[pix * 3 + 1] = acc.cg;
    out_rgb[pix * 3 + 2] = acc.cb;
    out_alpha[pix] = 1.f - acc.trans;
  }
  if (__ballot(bad) != 0ull && l == 0) atomicExch(status, 1);
  if (counters && l == 0) {
    atomicAdd(counters + 1, (unsigned long long)n_proc);
    atomicAdd(counters + 2, (unsigned long long)n_proc_hit);
    atomicAdd(counters + 3, (unsigned long long)n_hits);
  }
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_mfma_pack_bytes(int num_primitives) {
  return num_primitives < 0 ? 0 : (size_t)(num_primitives > 0 ? num_primitives : 1) * kPackStride;
}

MLPSP_API int mlpsp_pack_mfma_weights(const float* W1, const float* b1, const float* W2, const float* b2,
                                      const float* W3, const float* b3, int num_primitives, int use_bf16,
                                      void* packed_dev, mlpsp_stream_t stream) {
  if (num_primitives < 0) return MLPSP_E_ARGUMENT;
  if (num_primitives == 0) return MLPSP_OK;
  if (!W1 || !b1 || !W2 || !b2 || !W3 || !b3 || !packed_dev) return MLPSP_E_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(packed_dev) % 128 != 0) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (use_bf16)
    hipLaunchKernelGGL(pack_mfma_weights_kernel<__bf16>, dim3(num_primitives), dim3(64), 0, s, W1, b1, W2, b2, W3, b3,
                       num_primitives, (unsigned char*)packed_dev);
  else
    hipLaunchKernelGGL(pack_mfma_weights_kernel<_Float16>, dim3(num_primitives), dim3(64), 0, s, W1, b1, W2, b2, W3, b3,
                       num_primitives, (unsigned char*)packed_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_render_tilecenter_mfma(const float* rays_o_dev, const float* rays_d_dev,
                                           const void* prim_records_dev, const int32_t* order_dev,
                                           const int32_t* tile_offsets_dev, const float* freq_dev,
                                           const float* att_dev, const void* packed_dev, int num_primitives,
                                           int use_bf16, int width, int height, float threshold, float* out_rgb_dev,
                                           float* out_alpha_dev, int32_t* status_dev, int64_t* counters_dev,
                                           mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, 8, 8);
  if (T <= 0 || T > 2147483647LL - 8 || num_primitives < 0) return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !freq_dev || !att_dev || !out_rgb_dev || !out_alpha_dev ||
      !status_dev)
    return MLPSP_E_ARGUMENT;
  if (num_primitives > 0 && !packed_dev) return MLPSP_E_ARGUMENT;
  MLPSP_HIP_TRY(hipMemsetAsync(status_dev, 0, 16 * sizeof(int32_t), (hipStream_t)stream));
  const int per_xcd = (int)((T + kNumXcd - 1) / kNumXcd);
  const dim3 grid((unsigned)(per_xcd * kNumXcd)), block(64);
  hipStream_t s = (hipStream_t)stream;
  auto* ctr = reinterpret_cast<unsigned long long*>(counters_dev);
  const int ntx = ceil_div(width, 8);
  if (use_bf16)
    hipLaunchKernelGGL(render_tilecenter_mfma_kernel<__bf16>, grid, block, 0, s, rays_o_dev, rays_d_dev,
                       (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,
                       (const unsigned char*)packed_dev, num_primitives, width, height, ntx, per_xcd, (int)T, threshold,
                       out_rgb_dev, out_alpha_dev, status_dev, ctr);
  else
    hipLaunchKernelGGL(render_tilecenter_mfma_kernel<_Float16>, grid, block, 0, s, rays_o_dev, rays_d_dev,
                       (const PrimRecord*)prim_records_dev, order_dev, tile_offsets_dev, freq_dev, att_dev,
                       (const unsigned char*)packed_dev, num_primitives, width, height, ntx, per_xcd, (int)T, threshold,
                       out_rgb_dev, out_alpha_dev, status_dev, ctr);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
