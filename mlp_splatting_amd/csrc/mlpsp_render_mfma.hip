// libmlpsp_hip: tile-centre-order forward render with the 72->32->32->4 MLP on the matrix cores.
//
// Counterpart of the reference's tensor-core kernel (scannet/cuda/rgb_wmma.cuh:75-223): geometry,
// activations and compositing stay f32; encoded inputs, weights and hidden activations are rounded
// to bf16 (or fp16) and multiplied with v_mfma_f32_32x32x16 with f32 accumulation.
//
// One wavefront = one 8x8 tile = 64 pixels; the MLP of a hit runs as mlp_wave_mfma16 (mlpsp_mfma16.hpp:
// transposed GEMMs, weights as the A operand in a layout packed once per scene by the kernel below, no LDS
// or cross-lane traffic between the layers).  (Measured alternatives that did not pay on gfx950: a
// 4096-entry LDS sin/cos table -- same kernel time, 2x the image error; persistent wavefronts with a tile
// work queue -- 6 % slower than one wavefront per tile.)
#include "mlpsp_device.hpp"
#include "mlpsp_hitrec.hpp"
#include "mlpsp_mfma16.hpp"
#include "mlpsp_host.hpp"

// 32-channel accumulator tiles per wavefront of the feature GEMM: a block of four wavefronts covers 128 x this many
// channels of a tile (2: three blocks per CU instead of two, a few percent faster than 4 on 512 channels)
#ifndef MLPSP_GEMM_NCB
#define MLPSP_GEMM_NCB 2
#endif

namespace mlpsp {

// ---------------------------------------------------------------------------------------------
// pack: f32 [N,32,72] [N,32] [N,32,32] [N,32] [N,4,32] [N,4]  ->  N blocks of kPackStride bytes
// ---------------------------------------------------------------------------------------------
// S: the type the six tensors are stored in (float, or _Float16 for an inference export read without widening it first:
// every fp16 value is an f32 value, so both sources give the same blocks bit for bit).
template <typename T, typename S>
__global__ __launch_bounds__(64) void pack_mfma_weights_kernel(const S* __restrict__ W1, const S* __restrict__ b1,
                                                               const S* __restrict__ W2, const S* __restrict__ b2,
                                                               const S* __restrict__ W3, const S* __restrict__ b3,
                                                               int N, unsigned char* __restrict__ out) {
  const int p = blockIdx.x;
  if (p >= N) return;
  const int l = threadIdx.x, m = l & 31, g = l >> 5;
  unsigned char* blk = out + (size_t)p * kPackStride;
  // accumulator row m holds hidden unit hidden_unit_of_row(m), for both hidden layers
  const S* w1 = W1 + (size_t)p * 32 * 72 + hidden_unit_of_row(m) * 72;
  const S* w2 = W2 + (size_t)p * 32 * 32 + hidden_unit_of_row(m) * 32;
  bool bad = false;
  auto pk = [&](float a, float b) {
    bad |= !(__builtin_fabsf(Ops<T>::round_trip(a)) <= Ops<T>::kMax) || !(__builtin_fabsf(Ops<T>::round_trip(b)) <= Ops<T>::kMax);
    return Ops<T>::pack2(a, b);
  };
  const float bias1 = (float)b1[(size_t)p * 32 + hidden_unit_of_row(m)], bias2 = (float)b2[(size_t)p * 32 + hidden_unit_of_row(m)];
  bad |= !(__builtin_fabsf(Ops<T>::round_trip(bias1)) <= Ops<T>::kMax) || !(__builtin_fabsf(Ops<T>::round_trip(bias2)) <= Ops<T>::kMax);
  for (int s = 0; s < 5; ++s) {
    u32x4 v;
    for (int d = 0; d < 4; ++d) {
      const int t = 4 * s + d;
      float ws = 0.f, wc = 0.f;
      if (t < 18) {
        const int j = (t / 3) * 6 + 3 * g + (t % 3);
        ws = (float)w1[j];
        wc = (float)w1[36 + j];
      }
      v[d] = pk(ws, wc);
      if (t == 18 && g == 0) v[d] = bias_word<T>(bias1);     // multiplied by the constant (1, 1) operand word
      if (t == 19 && g == 0) v[d] = bias_word<T>(bias2);     // by zero in layer 1, by (1, 1) in layer 2's bias step
    }
    *reinterpret_cast<u32x4*>(blk + kOffW1 + s * 1024 + l * 16) = v;
  }
  for (int s = 0; s < 2; ++s) {
    u32x4 v;
    for (int d = 0; d < 4; ++d) v[d] = pk((float)w2[hidden_unit(8 * s + 2 * d, g)], (float)w2[hidden_unit(8 * s + 2 * d + 1, g)]);
    *reinterpret_cast<u32x4*>(blk + kOffW2 + s * 1024 + l * 16) = v;
  }
  reinterpret_cast<unsigned*>(blk + kOffB2)[l] = 0u;         // reserved
  if (l < 16) {
    const int row = l & 3, gg = (l >> 2) & 1, s = l >> 3;
    const S* w3 = W3 + (size_t)p * 4 * 32 + row * 32;
    u32x4 v;
    for (int d = 0; d < 4; ++d) v[d] = pk((float)w3[hidden_unit(8 * s + 2 * d, gg)], (float)w3[hidden_unit(8 * s + 2 * d + 1, gg)]);
    *reinterpret_cast<u32x4*>(blk + kOffW3 + ((s * 2 + gg) * 4 + row) * 16) = v;
  }
  if (l < 4) {
    const float v3 = (float)b3[(size_t)p * 4 + l];
    bad |= !(__builtin_fabsf(v3) <= 3.4028235e38f);
    reinterpret_cast<float*>(blk + kOffB3)[l] = v3;
  }
  const unsigned long long any = __ballot(bad);
  if (l == 0) *reinterpret_cast<int32_t*>(blk + kOffFlag) = any ? 1 : 0;
  if (l < (kPackStride - kOffFlag - 4) / 4) reinterpret_cast<unsigned*>(blk + kOffFlag + 4)[l] = 0u;   // unused tail
}

// ---------------------------------------------------------------------------------------------
// render
// ---------------------------------------------------------------------------------------------

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
__device__ __forceinline__ float fast_blend_step(PixelAcc& a, float o0, float o1, float o2, float o3, float decay) {
  const float sigma = fast_softplus(o3) * decay;
  const float alpha = 1.f - fast_exp(-sigma);
  const float w = a.trans * alpha;
  a.cr = fmaf(w, fast_sigmoid(o0), a.cr);
  a.cg = fmaf(w, fast_sigmoid(o1), a.cg);
  a.cb = fmaf(w, fast_sigmoid(o2), a.cb);
  a.trans = a.trans * (1.f - alpha);
  return w;
}
// tetrahedral gates (np_tile_kernels.cu:97-124) with the native exp/rcp.  qs = local hit offset divided by the
// scales (what hit_fast() returns); u = q / (beta s + 1e-6) = qs k with k = s / (beta s + 1e-6), which depends on
// the primitive alone (gate_factor).
__device__ __forceinline__ float gate_factor(float lg, float beta) {
  const float s = fast_exp(lg);
  return s * __builtin_amdgcn_rcpf(beta * s + 1e-6f);
}
__device__ __forceinline__ void fast_tetra_gates(float qsx, float qsy, float qsz, float kx, float ky, float kz,
                                                 float temp, float g[4]) {
  const float ux = fminf(1.f, fmaxf(-1.f, qsx * kx));
  const float uy = fminf(1.f, fmaxf(-1.f, qsy * ky));
  const float uz = fminf(1.f, fmaxf(-1.f, qsz * kz));
  const float l0 = temp * ((ux + uy) + uz), l1 = temp * ((ux - uy) - uz);
  const float l2 = temp * ((-ux + uy) - uz), l3 = temp * ((-ux - uy) + uz);
  const float lm = fmaxf(fmaxf(l0, l1), fmaxf(l2, l3));
  const float e0 = fast_exp(l0 - lm), e1 = fast_exp(l1 - lm), e2 = fast_exp(l2 - lm), e3 = fast_exp(l3 - lm);
  const float inv = __builtin_amdgcn_rcpf(fmaxf(((e0 + e1) + e2) + e3, 1e-8f));
  g[0] = e0 * inv;
  g[1] = e1 * inv;
  g[2] = e2 * inv;
  g[3] = e3 * inv;
}

// The second half of a PrimRecord (mlpsp_device.hpp): one 64-byte line per primitive.
struct FastRec {
  float cx, cy, cz;
  float r[9];
  float pad[4];
};
static_assert(sizeof(FastRec) == 64, "second half of PrimRecord");

// The 12 floats of a FastRec as scalar registers, requested with explicit scalar loads so that the request sits
// exactly where it is written (the compiler otherwise sinks such a load to its first use, which is the next
// loop iteration: every candidate would then wait for its own record).  fast_arrived() must run before the
// registers are read; waits the compiler inserts for its own scalar and LDS operations in between only wait
// longer for having one more operation outstanding.
typedef float f32x8 __attribute__((ext_vector_type(8)));
struct FastRegs {
  f32x4 a;   // cx cy cz r0
  f32x8 b;   // r1 .. r8
};
__device__ __forceinline__ void fast_request(const unsigned char* __restrict__ line, FastRegs& q) {
  asm volatile("s_load_dwordx4 %0, %2, 0x0\n\ts_load_dwordx8 %1, %2, 0x10" : "=&s"(q.a), "=&s"(q.b) : "s"(line));
}
__device__ __forceinline__ FastRec fast_arrived(FastRegs& q) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(q.a), "+s"(q.b));
  FastRec F;
  F.cx = q.a[0]; F.cy = q.a[1]; F.cz = q.a[2];
  F.r[0] = q.a[3];
#pragma unroll
  for (int k = 0; k < 8; ++k) F.r[1 + k] = q.b[k];
  return F;
}

// Ray against rotated ellipsoid for this path: same quantities as hit_rot() (np_tile_kernels.cu:659-711), with
// the world -> local rotation and the inverse scales applied as one matrix, the local hit offset taken as
// vl - t dl (equal to the rotated world offset up to rounding), and the native reciprocal and exp2.  About a
// third of the instructions of the exactly-rounded form; the differences are of the order of f32 rounding of
// the long vector vl (how large: below).  h.ql* are in units of the scales.
//
// The hit decision itself is a hard threshold, and a primitive that barely hits still contributes up to a
// few 1e-3 to a pixel, so a decision that differs from the exact path's would show as isolated pixel
// errors well above the rounding noise of this path.  unsure = the fast quantities are too close to one of
// the three decision boundaries (decay within `band` of thr, t or denom near zero) to be trusted; the
// caller then takes the decision -- only the decision -- from hit_rot().
//
// How wide the band has to be: with u = 2^-24, vl and dl carry about 4 u |vl| and 4 u |dl| of rounding (entries of
// r rounded, three-term sums), t = numer / denom about 24 u |vl| / |dl|, so ql = vl - t dl is off by up to
// 32 u |vl| and r2 = |ql|^2 by 64 u |ql| |vl|, i.e. ln decay by 32 u |ql| |vl|, and the exactly rounded form,
// which rotates the same long vector, by as much again: 64 u |ql| |vl| = 3.8e-6 |ql| |vl| relative in decay, with
// |ql| = sqrt(-2 ln thr) at the threshold (3.3 for thr = 5e-3: 1.3e-5 |vl|) and |vl| = distance origin -> centre
// in units of the scales (a hundred is typical, far small primitives reach thousands).  band_for() is that
// bound plus a floor for the native exp2; reach = 4e-6 sqrt(-2 ln thr).
// What hit_fast() needs of (primitive, ray origin) alone: the offset centre - origin and its image under r.
struct OriginTerms {
  float vx, vy, vz, vlx, vly, vlz;
};
__device__ __forceinline__ float band_for(const OriginTerms& o, float thr, float reach) {
  const float len = __builtin_amdgcn_sqrtf(fmaf(o.vlx, o.vlx, fmaf(o.vly, o.vly, o.vlz * o.vlz)));   // (one ulp is plenty)
  return thr * fmaf(reach, len, 3e-5f);
}
__device__ __forceinline__ OriginTerms origin_terms(float ox, float oy, float oz, float cx, float cy, float cz,
                                                    const float r[9]) {
  OriginTerms o;
  o.vx = cx - ox;
  o.vy = cy - oy;
  o.vz = cz - oz;
  o.vlx = fmaf(r[0], o.vx, fmaf(r[1], o.vy, r[2] * o.vz));
  o.vly = fmaf(r[3], o.vx, fmaf(r[4], o.vy, r[5] * o.vz));
  o.vlz = fmaf(r[6], o.vx, fmaf(r[7], o.vy, r[8] * o.vz));
  return o;
}
__device__ __forceinline__ bool hit_fast(const OriginTerms& o, float rdx, float rdy, float rdz, const float r[9],
                                         float thr, float band, HitInfo& h, bool& unsure) {
  const float dlx = fmaf(r[0], rdx, fmaf(r[1], rdy, r[2] * rdz));
  const float dly = fmaf(r[3], rdx, fmaf(r[4], rdy, r[5] * rdz));
  const float dlz = fmaf(r[6], rdx, fmaf(r[7], rdy, r[8] * rdz));
  const float denom = fmaf(dlx, dlx, fmaf(dly, dly, dlz * dlz));
  const float numer = fmaf(dlx, o.vlx, fmaf(dly, o.vly, dlz * o.vlz));
  const float t = numer * __builtin_amdgcn_rcpf(denom);
  h.t = t;
  h.dx = fmaf(-t, rdx, o.vx);
  h.dy = fmaf(-t, rdy, o.vy);
  h.dz = fmaf(-t, rdz, o.vz);
  h.qlx = fmaf(-t, dlx, o.vlx);
  h.qly = fmaf(-t, dly, o.vly);
  h.qlz = fmaf(-t, dlz, o.vlz);
  const float r2 = fmaf(h.qlx, h.qlx, fmaf(h.qly, h.qly, h.qlz * h.qlz));
  h.decay = __builtin_amdgcn_exp2f(r2 * -0.72134752f);
  unsure = (__builtin_fabsf(h.decay - thr) <= band) || !(__builtin_fabsf(t) >= 1e-4f) || !(denom >= 1e-18f);
  return !(denom <= 1e-20f) && !(t <= 0.f) && (h.decay > thr);
}

// LDS of one wavefront: the OriginTerms of the 64 list entries it is walking and the width of their decision
// band (one address register for the two reads of a step); with a gated feature channel also the entries' three
// gate factors, which a hit would otherwise have to fetch from the primitive's record -- a load that nothing but
// the gates waits for, at the end of the step.
template <int SP>
struct OriginLds {
  float e[64][SP > 0 ? 12 : 8];
};

// The table only for bf16 operands (see kSinCosEntries).
template <typename T> struct RenderTable { static constexpr bool kUse = false; unsigned w[1]; };
#if !defined(MLPSP_RENDER_NO_TABLE)
template <> struct RenderTable<__bf16> { static constexpr bool kUse = true; SinCosTable t; };
#endif

// SP = 0: RGB only.  SP = 4 or 8: the kernel also emits, per tile, the compact list of primitives that
// hit at least one pixel (hit records, mlpsp_hitrec.hpp) and per (such primitive, pixel) the SP compositing
// coefficients of the gated feature channel, rounded to fp16 (they lie in [0, 1]; fp16 keeps 11
// significant bits there, bf16 only 8): (w g0, w g1, w g2, w g3) for 4 slots,
// (w, 0, 0, 0) for one slot, (w, w g0, .., w g3, 0, 0, 0) for 5 slots (np_tile_kernels.cu:6036-6075:
// feat += w * (base + sum_s g_s attr_s)).  The feature image is then one grouped GEMM over those lists
// (feat_gemm_kernel below).
// Register budget: 128 VGPRs, i.e. four wavefronts per SIMD (a dozen values spill; measured 4.5 % faster
// than the 146 registers and three wavefronts the compiler picks on its own).
// One tile, rendered by the calling wavefront (lane l = pixel l of the tile); s_dir: LDS of this wavefront alone.
template <typename T, int SP>
__device__ __forceinline__ void render_tile_mfma(
    const int tile, const int l, DirWords& s_dir, OriginLds<SP>& s_org, const SinCosTable* table,
    const float* __restrict__ rays_o,
    const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims, const int32_t* __restrict__ order, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ ends,
    const float* __restrict__ freq, const float* __restrict__ att, const unsigned char* __restrict__ packed, int N,
    int W, int H, int ntx, float thr, float* __restrict__ out_rgb, float* __restrict__ out_alpha,
    int32_t* __restrict__ status, unsigned long long* __restrict__ counters, int slots, float beta, float temp,
    const HitPool& hp) {
  float kf[3];
  phase_scales(freq, att, l >> 5, kf);
  // With the sin/cos table the MLP takes its phase scales in units of a quarter table entry, and the inputs must
  // stay below kSinCosRange revolutions at the highest frequency (else the frame is flagged and rendered in f32,
  // like any other operand this path cannot represent).
  float kfm[3] = {kf[0], kf[1], kf[2]};
  float input_limit = 3.4028235e38f;
  if constexpr (RenderTable<T>::kUse) {
    float kmax = fmaxf(fmaxf(__builtin_fabsf(kf[0]), __builtin_fabsf(kf[1])), __builtin_fabsf(kf[2]));
    kmax = fmaxf(kmax, __shfl_xor(kmax, 32));
    input_limit = kSinCosRange / fmaxf(kmax, 1e-30f);
#pragma unroll
    for (int j = 0; j < 3; ++j) kfm[j] = kf[j] * (4.0f * (float)kSinCosEntries);
  }
  unsigned n_proc = 0, n_proc_hit = 0, n_hits = 0;
  bool bad = false;
  const int tx = tile % ntx, ty = tile / ntx;
  const int x = tx * 8 + (l & 7), y = ty * 8 + (l >> 3);
  const bool valid = (x < W) && (y < H);
  const int pix = valid ? (y * W + x) : 0;
  const Float3 ray_o = valid ? load3(rays_o, pix) : Float3{0.f, 0.f, 0.f};
  const Float3 ray_d = valid ? load3(rays_d, pix) : Float3{0.f, 0.f, 0.f};
  const float rox = ray_o.x, roy = ray_o.y, roz = ray_o.z;
  const float rdx = ray_d.x, rdy = ray_d.y, rdz = ray_d.z;
  // The encoding of the ray direction (input components 0..2, operand words 0..8 of both column blocks) does
  // not depend on the primitive: it is computed once per pixel and parked in LDS in operand form -- 18 more
  // live registers would cost the fourth wavefront per SIMD.  Written and read by this wavefront only: no barrier.
  encode_direction_words<T>(rdx, rdy, rdz, kf, l, s_dir);

  // A tile whose rays start from one point (a pinhole camera: every tile) needs centre - origin and its rotated,
  // scaled image once per list entry, not once per pixel: lane j works them out for entry j of the 64 the wavefront
  // is about to walk and parks them in LDS; a step then reads them with two broadcast reads instead of twelve
  // vector instructions.  Same expressions on the same operands as the per-pixel form, so the same bits.
  const unsigned long long in_image = __ballot(valid);
  const int lane0 = in_image ? (int)__builtin_ctzll(in_image) : 0;
  const float ox = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(rox), lane0)),
              oy = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(roy), lane0)),
              oz = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(roz), lane0));
  const float reach = 4e-6f * __builtin_sqrtf(fmaxf(-2.f * __logf(thr), 0.f));   // see band_for()
  const bool one_origin = __ballot(valid && !(rox == ox && roy == oy && roz == oz)) == 0ull;

  const int start = offsets[tile], end = ends[tile];
  PixelAcc acc = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
  HitEmitter em = hit_emitter_begin(hp, 0, start, tile);
  bool live = valid;
  const unsigned char* __restrict__ fast_half = reinterpret_cast<const unsigned char*>(prims) + 64;

  // The tile's list is read 64 entries at a time, one coalesced load; a lane's entry is broadcast with
  // v_readlane when its turn comes.  Culled (negative) entries never get a turn.  The geometry line of the next
  // entry is requested as soon as the current one has been tested -- ahead of its MLP, if it hit -- so that neither
  // the id nor the record is waited for long in a run of candidates that hit nothing.
  bool finished = false;
  for (int base = start; base < end && !finished; base += 64) {
    const int id_lane = (base + l < end) ? order[base + l] : -1;
    unsigned long long todo = __ballot(id_lane >= 0 && id_lane < N);
    if (todo == 0ull) continue;
    if (one_origin && id_lane >= 0 && id_lane < N) {
      const FastRec& F = *reinterpret_cast<const FastRec*>(fast_half + (size_t)id_lane * sizeof(PrimRecord));
      const OriginTerms o = origin_terms(ox, oy, oz, F.cx, F.cy, F.cz, F.r);
      *reinterpret_cast<f32x4*>(&s_org.e[l][0]) = f32x4{o.vx, o.vy, o.vz, o.vlx};
      *reinterpret_cast<f32x4*>(&s_org.e[l][4]) = f32x4{o.vly, o.vlz, band_for(o, thr, reach), 0.f};
    }
    if constexpr (SP > 0) {
      if (slots > 1 && id_lane >= 0 && id_lane < N) {
        const PrimRecord& P = prims[id_lane];
        *reinterpret_cast<f32x4*>(&s_org.e[l][8]) =
            f32x4{gate_factor(P.lgx, beta), gate_factor(P.lgy, beta), gate_factor(P.lgz, beta), 0.f};
      }
    }
    int j = (int)__builtin_ctzll(todo);
    int p = __builtin_amdgcn_readlane(id_lane, j);
    todo &= todo - 1ull;
    FastRegs q;
    fast_request(fast_half + (size_t)p * sizeof(PrimRecord), q);
    for (;;) {
      // Between fast_arrived() and the next fast_request() every use of R: the request reloads the same scalar
      // registers, and a value of R that had to outlive it would be copied out of them at the loop's edge, i.e.
      // while they are being loaded.
      const FastRec R = fast_arrived(q);
      OriginTerms ot;
      float band;
      if (one_origin) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(&s_org.e[j][0]);
        const f32x4 b = *reinterpret_cast<const f32x4*>(&s_org.e[j][4]);
        ot = OriginTerms{a[0], a[1], a[2], a[3], b[0], b[1]};
        band = b[2];
      } else {
        ot = origin_terms(rox, roy, roz, R.cx, R.cy, R.cz, R.r);
        band = band_for(ot, thr, reach);
      }
      HitInfo h;
      bool unsure;
      bool hit = hit_fast(ot, rdx, rdy, rdz, R.r, thr, band, h, unsure) && live;
      asm volatile("" : "+v"(h.t), "+v"(h.qlx), "+v"(h.qly), "+v"(h.qlz), "+v"(h.decay));   // R is used up here

      const bool more = todo != 0ull;
      int p_next = p, j_next = j;
      if (more) {
        j_next = (int)__builtin_ctzll(todo);
        p_next = __builtin_amdgcn_readlane(id_lane, j_next);
        todo &= todo - 1ull;
        // (only when an entry follows: a request nobody waits for would still be landing in these registers after
        // the loop, when the compiler has long given them to something else)
        fast_request(fast_half + (size_t)p_next * sizeof(PrimRecord), q);
      }
      if (__ballot(unsure && live) != 0ull) {   // rare
        if (unsure && live) {
          const PrimRecord P = prims[p];
          HitInfo exact;
          hit = hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, exact);
        }
      }
      const unsigned long long mask = __ballot(hit);
      ++n_proc;
      if (mask != 0ull) {
        ++n_proc_hit;
        n_hits += __popcll(mask);
        const unsigned char* __restrict__ blk = packed + (size_t)p * kPackStride;
        bad |= hit && !((__builtin_fabsf(h.dx) + __builtin_fabsf(h.dy)) + __builtin_fabsf(h.dz) <= input_limit);
        float o[4];
        if ((unsigned)mask != 0u && (unsigned)(mask >> 32) != 0u)
          bad |= mlp_pair_mfma16<T, Ops<T>::kCheckHidden, RenderTable<T>::kUse>(blk, mask, l, h.dx, h.dy, h.dz, kfm, s_dir, o,
                                                                               table);
        else
          bad |= mlp_wave_mfma16<T, Ops<T>::kCheckHidden, false, RenderTable<T>::kUse>(blk, mask, l, h.dx, h.dy, h.dz, kfm,
                                                                                      s_dir, o, nullptr, table);
        float w = 0.f;
        if (hit) {
          bad |= !(max3_abs(o[0], o[1], o[2]) <= 3.4028235e38f) || !(__builtin_fabsf(o[3]) <= 3.4028235e38f);
          w = fast_blend_step(acc, o[0], o[1], o[2], o[3], h.decay);
        }
        if constexpr (SP > 0) {
          float gt[4] = {0.f, 0.f, 0.f, 0.f};
          if (slots > 1) {
            const f32x4 k = *reinterpret_cast<const f32x4*>(&s_org.e[j][8]);
            if (hit) fast_tetra_gates(h.qlx, h.qly, h.qlz, k[0], k[1], k[2], temp, gt);
          }
          const int rs = hit_emitter_next(hp, em, l);
          if (rs >= 0) {
            unsigned* __restrict__ coef = reinterpret_cast<unsigned*>(hp.records + (size_t)rs * hp.record_bytes);
            if constexpr (SP == 4) {
              const unsigned c01 = (slots > 1) ? Ops<_Float16>::pack2(w * gt[0], w * gt[1]) : Ops<_Float16>::pack2(w, 0.f);
              const unsigned c23 = Ops<_Float16>::pack2(w * gt[2], w * gt[3]);
              *reinterpret_cast<uint2*>(coef + l * 2) = make_uint2(c01, c23);
            } else {
              const u32x4 c = {Ops<_Float16>::pack2(w, w * gt[0]), Ops<_Float16>::pack2(w * gt[1], w * gt[2]),
                               Ops<_Float16>::pack2(w * gt[3], 0.f), 0u};
              *reinterpret_cast<u32x4*>(coef + l * 4) = c;
            }
            if (l == 0) hp.hit_ids[rs] = p;
          }
        }
        live = valid && (acc.trans >= kTransmittanceFloor);
        if (__ballot(live) == 0ull) {
          finished = true;
          break;
        }
      }
      if (!more) break;
      p = p_next;
      j = j_next;
    }
  }

  if (valid) {
    store3(out_rgb, pix, acc.cr, acc.cg, acc.cb);
    out_alpha[pix] = 1.f - acc.trans;
  }
  if constexpr (SP > 0) {
    if (l == 0) hp.item_hits[tile] = em.count;
  }
  if (__ballot(bad) != 0ull && l == 0) atomicExch(status, 1);
  if (counters && l == 0) {
    atomicAdd(counters + 1, (unsigned long long)n_proc);
    atomicAdd(counters + 2, (unsigned long long)n_proc_hit);
    atomicAdd(counters + 3, (unsigned long long)n_hits);
  }
}

// Four wavefronts = four tiles per workgroup: they share nothing but the sin/cos table, which they fill together
// (sixteen transcendentals per thread) before each goes its own way.
#ifndef MLPSP_RENDER_WAVES
#define MLPSP_RENDER_WAVES 4
#endif
constexpr int kRenderWaves = MLPSP_RENDER_WAVES;
template <typename T, int SP>
__global__ __launch_bounds__(64 * kRenderWaves) __attribute__((amdgpu_waves_per_eu(4, 4))) void render_tilecenter_mfma_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const int32_t* __restrict__ ends,
    const float* __restrict__ freq,
    const float* __restrict__ att, const unsigned char* __restrict__ packed, int N, int W, int H, int ntx,
    int per_xcd, int num_tiles, float thr, float* __restrict__ out_rgb, float* __restrict__ out_alpha,
    int32_t* __restrict__ status, unsigned long long* __restrict__ counters, int slots, float beta, float temp,
    HitPool hp) {
  __shared__ DirWords s_dir[kRenderWaves];
  __shared__ __attribute__((aligned(16))) OriginLds<SP> s_org[kRenderWaves];
  __shared__ RenderTable<T> s_table;
  const SinCosTable* table = nullptr;
  if constexpr (RenderTable<T>::kUse) {
    fill_sincos_table<T>(s_table.t);
    __syncthreads();
    table = &s_table.t;
  }
  // 8x8 super-blocks of tiles dealt to the XCDs in turn: neighbouring tiles, which share most primitives (their
  // records and weight blocks), run on one L2.  Workgroup b runs on XCD b % 8 and takes four consecutive slots of it.
  const int wave = (int)threadIdx.x >> 6;
  const int tile = superblock_tile_of((int)(blockIdx.x % kNumXcd), (int)(blockIdx.x / kNumXcd) * kRenderWaves + wave, ntx,
                                      num_tiles / ntx);
  if (tile < 0) return;
  render_tile_mfma<T, SP>(tile, (int)threadIdx.x & 63, s_dir[wave], s_org[wave], table, rays_o, rays_d, prims, order, offsets,
                          ends, freq, att, packed, N, W, H, ntx, thr, out_rgb, out_alpha, status, counters, slots, beta, temp,
                          hp);
}

// ---------------------------------------------------------------------------------------------
// feature channel: pack + grouped GEMM
// ---------------------------------------------------------------------------------------------

// feat_attr f32 [N, S, C] (S = 1: [N, C])  ->  fp16 [N, C, SP] (the reference's inference export stores
// these attributes as fp16 too, scannet/cumodel.py:317-381), the SP slot values of one (primitive, channel)
// contiguous (slot order as the coefficient records above, zero padded).  flag[0] = 1 if a rounded value
// is not finite.
template <int SP, typename SRC>
__global__ __launch_bounds__(256) void pack_feat_kernel(const SRC* __restrict__ attr, int N, int S, int C,
                                                        unsigned* __restrict__ out, int32_t* __restrict__ flag) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)N * C) return;
  const size_t p = idx / C;
  const int c = (int)(idx % C);
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  bool bad = false;
  for (int s = 0; s < S; ++s) {
    v[s] = (float)attr[(p * S + s) * C + c];
    bad |= !(__builtin_fabsf(Ops<_Float16>::round_trip(v[s])) <= Ops<_Float16>::kMax);
  }
#pragma unroll
  for (int d = 0; d < SP / 2; ++d) out[idx * (SP / 2) + d] = Ops<_Float16>::pack2(v[2 * d], v[2 * d + 1]);
  if (bad) atomicExch(flag, 1);
}

// out_feat[pixel, c] = sum over the tile's hit records e and slots s of coef[e, pixel, s] * attr[id_e, c, s]:
// per tile a [64 pixels] x [K = SP * hits] x [C] product on v_mfma_f32_32x32x16.  One 256-thread block per
// (tile, slice of 128 NCB channels); wavefront v owns channels [128 v, 128 v + 128) of the slice as 2 pixel blocks
// x 4 channel blocks of f32 accumulators (NCB = 4).  Pixels are the M operand and channels the N operand, so
// that an accumulator register holds 32 consecutive channels of one pixel across lanes: every store is a full
// 128-byte line.
//
// The product is bound by the latency of its operand loads, not by the matrix cores (13 K-steps per tile on
// average, each needing 4 KB of attributes per record from L2), so the operands go through LDS in chunks of
// kGemmChunk records: all 256 threads request the chunk's attribute rows (the block's channel slice, up to 4 KB per
// record for 4 slots) and its coefficient records (contiguous in the pool: a pool chunk is kHitChunk records) at
// once -- ten or more 16-byte loads in flight per thread instead of one K-step's -- then write them to LDS, and
// after a barrier the wavefronts multiply out of LDS (8-byte or 16-byte reads, lanes on consecutive addresses).
// Two or three blocks share a CU, so one block's loads overlap another's multiplications and stores.  (Holding the
// next chunk's loads in registers across the multiplication measured slower: the registers cost a block per CU.)
// K-slot j of lane group g is (record 16/SP * step + g * 8/SP + j / SP, slot j % SP).
template <int SP>
struct GemmChunk {
  static constexpr int kRecords = 64 / SP;      // 16 records of 4 slots, 8 records of 8: K = 64 per chunk
};

template <int SP, int NCB>
__global__ __launch_bounds__(256) void feat_gemm_kernel(const unsigned* __restrict__ attr, HitPool hp,
                                                        const int32_t* __restrict__ offsets, int C, int W, int H,
                                                        int ntx, int per_xcd, int num_tiles,
                                                        float* __restrict__ out_feat) {
  // super-blocks of 8x8 tiles per XCD, as in the render: the 64 tiles that run together on an XCD are neighbours,
  // and a primitive's attribute row is fetched into that L2 once for all of them
  const int tile = superblock_tile(blockIdx.x, ntx, num_tiles / ntx);
  if (tile < 0) return;
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, g = l >> 5, m = l & 31;
  constexpr int EPL = 8 / SP;         // records per lane group and K-step
  constexpr int STEP = 2 * EPL;       // records per K-step (one MFMA per accumulator tile)
  constexpr int DW = SP / 2;          // dwords per (record, pixel) and per (primitive, channel)
  constexpr int R = GemmChunk<SP>::kRecords;
  constexpr int kSlice = 128 * NCB;   // channels per block
  constexpr int kRowDw = kSlice * DW; // dwords of one record's attribute row slice in LDS
  constexpr int kCoefDw = 64 * DW;    // dwords of one coefficient record
  constexpr int kStage = 512;         // records whose pool slot and primitive id are staged in LDS at a time
  static_assert(kHitChunk % R == 0, "a chunk of the product lies inside one chunk of the record pool");
  __shared__ __attribute__((aligned(16))) unsigned s_b[R * kRowDw];
  __shared__ __attribute__((aligned(16))) unsigned s_a[R * kCoefDw];
  __shared__ int s_slot[kStage / R];  // pool slot of the first record of each staged chunk
  __shared__ int s_prim[kStage];
  const int slice0 = (int)blockIdx.y * kSlice;           // first channel of the block
  const int c0 = slice0 + wave * (32 * NCB);
  const bool active = c0 < C;              // a wavefront without channels still helps staging and meets the barriers
  const int ncb = active ? min(NCB, (C - c0 + 31) / 32) : 0;
  const int hits = hp.item_hits[tile];
  const int table_base = (offsets[tile] >> 4) + tile;
  f32x16 acc[2][NCB];
#pragma unroll
  for (int pb = 0; pb < 2; ++pb)
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[pb][cb][r] = 0.f;

  // dwords of an attribute row that belong to this block's slice and exist: [0, row_dw)
  const int row_dw = min(kSlice, C - slice0) * DW;
  const bool wide = ((C * DW) & 3) == 0;                // rows start on 16-byte boundaries
  constexpr int kBLoads = R * kRowDw / 4 / 256;          // 16-byte pieces of the chunk's rows per thread
  constexpr int kALoads = R * kCoefDw / 4 / 256;         // ... of its coefficient records
  static_assert(kBLoads * 256 * 4 == R * kRowDw && kALoads * 256 * 4 == R * kCoefDw, "whole pieces per thread");

  for (int base = 0; base < hits; base += kStage) {
    const int n = min(kStage, hits - base);
    // record -> primitive id (and chunk -> pool slot) once per block, so that the chunk loop below has a single
    // level of global loads to wait for
    for (int k = threadIdx.x; k < n; k += 256) {
      const int rs = hit_slot(hp, table_base, base + k);
      if ((k & (R - 1)) == 0) s_slot[k / R] = rs;
      s_prim[k] = hp.hit_ids[rs];
    }
    __syncthreads();
    // requests chunk e0 of the staged records into registers (records past the end of the list as zeros)
    auto request = [&](int e0, u32x4 (&vb)[kBLoads], u32x4 (&va)[kALoads]) {
      const int nrec = min(R, n - e0);
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        const int piece = threadIdx.x + 256 * i;           // 16-byte piece of the chunk's row slices
        const int rec = piece / (kRowDw / 4), dw = (piece % (kRowDw / 4)) * 4;
        vb[i] = u32x4{0u, 0u, 0u, 0u};
        if (rec < nrec && dw < row_dw) {
          const unsigned* __restrict__ src = attr + ((size_t)s_prim[e0 + rec] * C + slice0) * DW + dw;
          if (wide && dw + 3 < row_dw) {
            vb[i] = *reinterpret_cast<const u32x4*>(src);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (dw + j < row_dw) vb[i][j] = src[j];
          }
        }
      }
      const unsigned* __restrict__ coef =
          reinterpret_cast<const unsigned*>(hp.records + (size_t)s_slot[e0 / R] * hp.record_bytes);
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        const int piece = threadIdx.x + 256 * i;
        va[i] = (piece / (kCoefDw / 4) < nrec) ? *reinterpret_cast<const u32x4*>(coef + piece * 4) : u32x4{0u, 0u, 0u, 0u};
      }
    };
    for (int e0 = 0; e0 < n; e0 += R) {
      const int nrec = min(R, n - e0);
      u32x4 vb[kBLoads], va[kALoads];
      request(e0, vb, va);
      // ---- into LDS
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<u32x4*>(&s_b[(threadIdx.x + 256 * i) * 4]) = vb[i];
#pragma unroll
      for (int i = 0; i < kALoads; ++i) *reinterpret_cast<u32x4*>(&s_a[(threadIdx.x + 256 * i) * 4]) = va[i];
      __syncthreads();
      // ---- multiply
      if (active) {
#pragma unroll
        for (int ks = 0; ks < R / STEP; ++ks) {
          if (ks * STEP >= nrec) break;
          u32x4 apix[2], bch[NCB];
#pragma unroll
          for (int u = 0; u < EPL; ++u) {
            const int rec = ks * STEP + g * EPL + u;
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
              const unsigned* pa = &s_a[rec * kCoefDw + (pb * 32 + m) * DW];
              if constexpr (SP == 4) {
                const uint2 v = *reinterpret_cast<const uint2*>(pa);
                apix[pb][2 * u] = v.x;
                apix[pb][2 * u + 1] = v.y;
              } else {
                apix[pb] = *reinterpret_cast<const u32x4*>(pa);
              }
            }
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
              const unsigned* pbch = &s_b[rec * kRowDw + (wave * (32 * NCB) + 32 * cb + m) * DW];
              if constexpr (SP == 4) {
                const uint2 v = *reinterpret_cast<const uint2*>(pbch);
                bch[cb][2 * u] = v.x;
                bch[cb][2 * u + 1] = v.y;
              } else {
                bch[cb] = *reinterpret_cast<const u32x4*>(pbch);
              }
            }
          }
#pragma unroll
          for (int cb = 0; cb < NCB; ++cb) {
            if (cb < ncb) {
#pragma unroll
              for (int pb = 0; pb < 2; ++pb) acc[pb][cb] = Ops<_Float16>::mfma(apix[pb], bch[cb], acc[pb][cb]);
            }
          }
        }
      }
      __syncthreads();
    }
  }
  if (!active) return;

  // The image is written through LDS: an accumulator register holds 32 consecutive channels of two pixels, i.e.
  // a store of it is two 128-byte lines, and the vector memory path takes as long for such an instruction as for
  // one that carries 16 bytes per lane.  Half a tile at a time every wavefront parks its accumulators in its own
  // quarter of the attribute chunk's LDS as [pixel][channel] (its 32 NCB channels of 32 pixels: 8 KB for NCB = 2)
  // and reads them back 16 bytes per lane, so that a store carries the wavefront's run of channels for 64 / (8 NCB)
  // pixels.  No workgroup barrier: a wavefront's LDS operations complete in order, and the chunk loop left every
  // wavefront behind its last barrier.
  constexpr int CW = 32 * NCB;             // channels of a wavefront
  constexpr int kLanesPerPixel = CW / 4, kPixelsPerStore = 64 / kLanesPerPixel;
  static_assert(sizeof(s_b) >= 4 * 32 * CW * sizeof(float), "four wavefronts' half tiles fit the attribute chunk");
  static_assert(kLanesPerPixel <= 64 && 64 % kLanesPerPixel == 0, "whole pixels per store");
  float* const s_t = reinterpret_cast<float*>(s_b) + wave * (32 * CW);
  const int tx = tile % ntx, ty = tile / ntx;
  const bool rows16 = (C & 3) == 0;        // a pixel's channels start on a 16-byte boundary
  const int cl = (l % kLanesPerPixel) * 4; // this lane's first channel within the wavefront's run
#pragma unroll
  for (int pb = 0; pb < 2; ++pb) {
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s_t[d_row(r, g) * CW + 32 * cb + m] = acc[pb][cb][r];
#pragma unroll
    for (int j = 0; j < 32 / kPixelsPerStore; ++j) {
      const int ql = j * kPixelsPerStore + l / kLanesPerPixel, q = 32 * pb + ql;
      const int x = tx * 8 + (q & 7), y = ty * 8 + (q >> 3);
      const f32x4 v = *reinterpret_cast<const f32x4*>(&s_t[ql * CW + cl]);
      if (x >= W || y >= H) continue;
      float* __restrict__ dst = out_feat + (size_t)(y * W + x) * C + c0 + cl;
      if (rows16 && c0 + cl + 3 < C) {
        *reinterpret_cast<f32x4*>(dst) = v;
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (c0 + cl + k < C) dst[k] = v[k];
      }
    }
  }
}

// Measurement aid: what the chip sustains on v_mfma_f32_32x32x16_bf16 when nothing else is in the way.
// Every wavefront runs `iterations` rounds of 8 independent accumulations on register operands.
__global__ __launch_bounds__(256) void probe_mfma_bf16_kernel(int iterations, float* __restrict__ sink) {
  u32x4 a = {0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u}, b = a;
  f32x16 acc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[k][r] = 0.f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = Ops<__bf16>::mfma(a, b, acc[k]);
  }
  float v = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) v += acc[k][0];
  if (v == 12345.678f) sink[0] = v;      // keeps the accumulations alive; practically never true
}

// Measurement aid: how do matrix-core, vector-ALU and transcendental instructions share a SIMD's issue time, inside
// one wavefront and across the wavefronts of a SIMD?  One workgroup of 16 wavefronts per CU (100 KB of dynamic LDS
// keeps a second one away): four wavefronts per SIMD, the render kernel's occupancy.  Every wavefront reads the SIMD
// it landed on from the hardware id register, takes a rank among that SIMD's wavefronts and with it one of the four
// roles the caller lists, runs the role's instruction batch over and over for a fixed stretch of the constant-rate
// clock, and reports how many batches it finished and how many core clocks passed.  Roles (instructions per batch):
//   0 idle   1 MFMA: 16 v_mfma_f32_32x32x16_bf16 on four independent accumulators   2 VALU: 128 independent v_fma_f32
//   3 transcendental: 128 v_sin_f32   4 mixed: 16 x (one MFMA, then eight v_fma_f32 that do not depend on it)
// The instructions are inline assembly so that the batches are exactly these sequences.
struct ProbeOut {
  long long batches, clocks;
  int role, simd;
};
#define MLPSP_PROBE_MFMA(acc) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define MLPSP_PROBE_FMA(x) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(m), "v"(c))
#define MLPSP_PROBE_SIN(x) asm volatile("v_sin_f32 %0, %0" : "+v"(x))
#define MLPSP_PROBE_8(OP) OP(v[0]); OP(v[1]); OP(v[2]); OP(v[3]); OP(v[4]); OP(v[5]); OP(v[6]); OP(v[7])

template <int ROLE>
__device__ __noinline__ long long probe_role(unsigned long long ticks, float* sink) {
  u32x4 a = {0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u}, b = a;
  f32x16 acc0, acc1, acc2, acc3;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = acc2[r] = acc3[r] = 0.f;
  float v[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] = 1e-3f * (float)(threadIdx.x + k);
  const float m = 1.0001f, c = 1e-3f * (float)threadIdx.x;
  long long batches = 0;
  const unsigned long long t0 = wall_clock64();
  while (wall_clock64() - t0 < ticks) {
    for (int rep = 0; rep < 4; ++rep) {
      if constexpr (ROLE == 0) __builtin_amdgcn_s_sleep(64);
      if constexpr (ROLE == 1)
        for (int i = 0; i < 4; ++i) { MLPSP_PROBE_MFMA(acc0); MLPSP_PROBE_MFMA(acc1); MLPSP_PROBE_MFMA(acc2); MLPSP_PROBE_MFMA(acc3); }
      if constexpr (ROLE == 2)
        for (int i = 0; i < 16; ++i) { MLPSP_PROBE_8(MLPSP_PROBE_FMA); }
      if constexpr (ROLE == 3)
        for (int i = 0; i < 16; ++i) { MLPSP_PROBE_8(MLPSP_PROBE_SIN); }
      if constexpr (ROLE == 4)
        for (int i = 0; i < 4; ++i) {
          MLPSP_PROBE_MFMA(acc0); MLPSP_PROBE_8(MLPSP_PROBE_FMA);
          MLPSP_PROBE_MFMA(acc1); MLPSP_PROBE_8(MLPSP_PROBE_FMA);
          MLPSP_PROBE_MFMA(acc2); MLPSP_PROBE_8(MLPSP_PROBE_FMA);
          MLPSP_PROBE_MFMA(acc3); MLPSP_PROBE_8(MLPSP_PROBE_FMA);
        }
      ++batches;
    }
  }
  asm volatile("s_nop 15\n s_nop 15\n s_nop 15");      // the accumulators are read below: let the last MFMA finish
  float r = 0.f;
  if constexpr (ROLE == 1 || ROLE == 4) r = (acc0[0] + acc1[1]) + (acc2[2] + acc3[3]);
#pragma unroll
  for (int k = 0; k < 8; ++k) r += v[k];
  if (r == 12345.678f) *sink = r;      // keeps the work alive; practically never true
  return batches;
}

__global__ __launch_bounds__(1024) void probe_issue_kernel(int r0, int r1, int r2, int r3, unsigned long long ticks,
                                                           ProbeOut* __restrict__ out, float* __restrict__ sink) {
  __shared__ int s_rank[4];
  if (threadIdx.x < 4) s_rank[threadIdx.x] = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int simd = (int)(__builtin_amdgcn_s_getreg((1 << 11) | (4 << 6) | 4) & 3u);   // HW_ID bits [5:4]
  int rank = 0;
  if (lane == 0) rank = atomicAdd(&s_rank[simd], 1);
  rank = __builtin_amdgcn_readfirstlane(rank) & 3;
  __syncthreads();
  const int role = rank == 0 ? r0 : rank == 1 ? r1 : rank == 2 ? r2 : r3;
  const long long c0 = clock64();
  long long batches = 0;
  switch (role) {
    case 1: batches = probe_role<1>(ticks, sink); break;
    case 2: batches = probe_role<2>(ticks, sink); break;
    case 3: batches = probe_role<3>(ticks, sink); break;
    case 4: batches = probe_role<4>(ticks, sink); break;
    default: batches = probe_role<0>(ticks, sink); break;
  }
  const long long c1 = clock64();
  if (lane == 0) out[blockIdx.x * 16 + (threadIdx.x >> 6)] = ProbeOut{batches, c1 - c0, role, simd};
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_mfma_pack_bytes(int num_primitives) {
  return num_primitives < 0 ? 0 : (size_t)(num_primitives > 0 ? num_primitives : 1) * kPackStride;
}

namespace {
template <typename S>
int pack_weights_from(const S* W1, const S* b1, const S* W2, const S* b2, const S* W3, const S* b3, int num_primitives,
                      int use_bf16, void* packed_dev, hipStream_t s) {
  if (num_primitives < 0) return MLPSP_E_ARGUMENT;
  if (num_primitives == 0) return MLPSP_OK;
  if (!W1 || !b1 || !W2 || !b2 || !W3 || !b3 || !packed_dev) return MLPSP_E_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(packed_dev) % 128 != 0) return MLPSP_E_ARGUMENT;
  if (use_bf16)
    hipLaunchKernelGGL((pack_mfma_weights_kernel<__bf16, S>), dim3(num_primitives), dim3(64), 0, s, W1, b1, W2, b2, W3,
                       b3, num_primitives, (unsigned char*)packed_dev);
  else
    hipLaunchKernelGGL((pack_mfma_weights_kernel<_Float16, S>), dim3(num_primitives), dim3(64), 0, s, W1, b1, W2, b2, W3,
                       b3, num_primitives, (unsigned char*)packed_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_pack_mfma_weights(const float* W1, const float* b1, const float* W2, const float* b2,
                                      const float* W3, const float* b3, int num_primitives, int use_bf16,
                                      void* packed_dev, mlpsp_stream_t stream) {
  return pack_weights_from<float>(W1, b1, W2, b2, W3, b3, num_primitives, use_bf16, packed_dev, (hipStream_t)stream);
}

MLPSP_API int mlpsp_pack_mfma_weights_half(const void* W1, const void* b1, const void* W2, const void* b2,
                                           const void* W3, const void* b3, int num_primitives, int use_bf16,
                                           void* packed_dev, mlpsp_stream_t stream) {
  typedef const _Float16* H;
  return pack_weights_from<_Float16>((H)W1, (H)b1, (H)W2, (H)b2, (H)W3, (H)b3, num_primitives, use_bf16, packed_dev,
                                     (hipStream_t)stream);
}

namespace {
constexpr int kGemmNcb = MLPSP_GEMM_NCB;   // 32-channel accumulator tiles per wavefront of the feature GEMM
constexpr size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
inline int feat_pad(int slots) { return slots == 5 ? 8 : 4; }

template <typename E, int SP>
void launch_mfma(dim3 grid, hipStream_t s, const float* rays_o, const float* rays_d, const void* prims, const int32_t* order,
                 const int32_t* offsets, const int32_t* ends, const float* freq, const float* att, const void* packed, int N, int W, int H,
                 int ntx, int per_xcd, int T, float thr, float* rgb, float* alpha, int32_t* status,
                 unsigned long long* ctr, int slots, float beta, float temp, const HitPool& hp) {
  hipLaunchKernelGGL((render_tilecenter_mfma_kernel<E, SP>), dim3(grid.x / kRenderWaves), dim3(64 * kRenderWaves), 0, s, rays_o, rays_d,
                     (const PrimRecord*)prims, order, offsets, ends, freq, att, (const unsigned char*)packed, N, W, H, ntx,
                     per_xcd, T, thr, rgb, alpha, status, ctr, slots, beta, temp, hp);
}
}  // namespace

MLPSP_API size_t mlpsp_mfma_feat_pack_bytes(int num_primitives, int feat_slots, int feat_channels) {
  if (num_primitives < 0 || feat_channels <= 0 || !(feat_slots == 1 || feat_slots == 4 || feat_slots == 5)) return 0;
  return align256((size_t)(num_primitives > 0 ? num_primitives : 1) * feat_channels * feat_pad(feat_slots) * 2);
}

namespace {
template <typename S>
int pack_feat_from(const S* feat_attr_dev, int num_primitives, int feat_slots, int feat_channels, void* packed_feat_dev,
                   int32_t* status_dev, hipStream_t s) {
  if (num_primitives < 0 || feat_channels <= 0 || feat_channels > 512 ||
      !(feat_slots == 1 || feat_slots == 4 || feat_slots == 5) || !status_dev)
    return MLPSP_E_ARGUMENT;
  MLPSP_HIP_TRY(hipMemsetAsync(status_dev, 0, sizeof(int32_t), s));
  if (num_primitives == 0) return MLPSP_OK;
  if (!feat_attr_dev || !packed_feat_dev || reinterpret_cast<uintptr_t>(packed_feat_dev) % 16 != 0) return MLPSP_E_ARGUMENT;
  const size_t total = (size_t)num_primitives * feat_channels;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  unsigned* out = (unsigned*)packed_feat_dev;
  if (feat_pad(feat_slots) == 4)
    hipLaunchKernelGGL((pack_feat_kernel<4, S>), grid, block, 0, s, feat_attr_dev, num_primitives, feat_slots,
                       feat_channels, out, status_dev);
  else
    hipLaunchKernelGGL((pack_feat_kernel<8, S>), grid, block, 0, s, feat_attr_dev, num_primitives, feat_slots,
                       feat_channels, out, status_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_pack_mfma_feat(const float* feat_attr_dev, int num_primitives, int feat_slots, int feat_channels,
                                   void* packed_feat_dev, int32_t* status_dev, mlpsp_stream_t stream) {
  return pack_feat_from<float>(feat_attr_dev, num_primitives, feat_slots, feat_channels, packed_feat_dev, status_dev,
                               (hipStream_t)stream);
}

MLPSP_API int mlpsp_pack_mfma_feat_half(const void* feat_attr_dev, int num_primitives, int feat_slots,
                                        int feat_channels, void* packed_feat_dev, int32_t* status_dev,
                                        mlpsp_stream_t stream) {
  return pack_feat_from<_Float16>((const _Float16*)feat_attr_dev, num_primitives, feat_slots, feat_channels,
                                  packed_feat_dev, status_dev, (hipStream_t)stream);
}

MLPSP_API int mlpsp_render_tilecenter_mfma_feat(const float* rays_o_dev, const float* rays_d_dev,
                                                const void* prim_records_dev, const int32_t* order_dev,
                                                const int32_t* tile_offsets_dev, int64_t num_pairs,
                                                const float* freq_dev, const float* att_dev, const void* packed_dev,
                                                int num_primitives, int use_bf16, const void* packed_feat_dev,
                                                int feat_slots, int feat_channels, float gating_beta,
                                                float gating_temp, int width, int height, float threshold,
                                                void* workspace_dev, size_t workspace_bytes, float* out_rgb_dev,
                                                float* out_alpha_dev, float* out_feat_dev, int32_t* status_dev,
                                                int64_t* counters_dev, int stage, const int32_t* tile_ends_dev,
                                                mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, 8, 8);
  if (stage < 0 || (stage & ~(3 | MLPSP_STAGE_STATUS_IS_CLEAR)) != 0) return MLPSP_E_ARGUMENT;
  const bool status_is_clear = (stage & MLPSP_STAGE_STATUS_IS_CLEAR) != 0;
  stage &= 3;
  if (stage > 2 || (stage != 0 && feat_slots == 0)) return MLPSP_E_ARGUMENT;
  if (T <= 0 || T > 2147483647LL - 8 || num_primitives < 0 || num_pairs < 0 || num_pairs > 2147483647LL)
    return MLPSP_E_ARGUMENT;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !freq_dev || !att_dev || !out_rgb_dev || !out_alpha_dev ||
      !status_dev)
    return MLPSP_E_ARGUMENT;
  if (num_primitives > 0 && !packed_dev) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  HitPool hp{};
  if (feat_slots != 0) {
    if (!(feat_slots == 1 || feat_slots == 4 || feat_slots == 5) || feat_channels <= 0 || feat_channels > 512 ||
        !out_feat_dev || (num_primitives > 0 && !packed_feat_dev))
      return MLPSP_E_ARGUMENT;
    if (!workspace_dev || reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0 ||
        workspace_bytes < hitpool_min_bytes(num_pairs, T, 1))
      return MLPSP_E_SCRATCH;
    hp = hitpool_carve(workspace_dev, workspace_bytes, num_pairs, T, 1, 64 * 2 * feat_pad(feat_slots));
    if (stage != 2) MLPSP_HIP_TRY(hipMemsetAsync(hp.counters, 0, 64 * sizeof(int32_t), s));
  }
  if (stage != 2 && !status_is_clear) MLPSP_HIP_TRY(hipMemsetAsync(status_dev, 0, 16 * sizeof(int32_t), s));
  const int per_xcd = (int)((T + kNumXcd - 1) / kNumXcd);
  const int ntx = ceil_div(width, 8);
  const int32_t* ends = tile_ends_dev ? tile_ends_dev : tile_offsets_dev + 1;
  const dim3 grid(superblock_grid(ntx, ceil_div(height, 8)));
  auto* ctr = reinterpret_cast<unsigned long long*>(counters_dev);
  const int sp = feat_slots ? feat_pad(feat_slots) : 0;
#define MLPSP_MFMA_GO(TT, SP)                                                                                     \
  launch_mfma<TT, SP>(grid, s, rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, ends, freq_dev,   \
                      att_dev, packed_dev, num_primitives, width, height, ntx, per_xcd, (int)T, threshold,        \
                      out_rgb_dev, out_alpha_dev, status_dev, ctr, feat_slots, gating_beta, gating_temp, hp)
#define MLPSP_MFMA_SP(TT)                 \
  do {                                    \
    if (sp == 0) MLPSP_MFMA_GO(TT, 0);    \
    else if (sp == 4) MLPSP_MFMA_GO(TT, 4); \
    else MLPSP_MFMA_GO(TT, 8);            \
  } while (0)
  if (stage != 2) {
    if (use_bf16) MLPSP_MFMA_SP(__bf16);
    else MLPSP_MFMA_SP(_Float16);
    MLPSP_LAUNCH_CHECK();
  }
#undef MLPSP_MFMA_SP
#undef MLPSP_MFMA_GO
  if (sp != 0 && stage != 1) {
    const dim3 ggrid(superblock_grid(ntx, ceil_div(height, 8)), (unsigned)ceil_div(feat_channels, 128 * kGemmNcb)), gblock(256);
#define MLPSP_FEAT_GEMM(SP)                                                                                       \
  hipLaunchKernelGGL((feat_gemm_kernel<SP, kGemmNcb>), ggrid, gblock, 0, s, (const unsigned*)packed_feat_dev, hp, \
                     tile_offsets_dev, feat_channels, width, height, ntx, per_xcd, (int)T, out_feat_dev)
    if (sp == 4) MLPSP_FEAT_GEMM(4);
    else MLPSP_FEAT_GEMM(8);
#undef MLPSP_FEAT_GEMM
    MLPSP_LAUNCH_CHECK();
    // status_dev[1] = 1 if the record pool was too small (the feature image is then incomplete)
    MLPSP_HIP_TRY(hipMemcpyAsync(status_dev + 1, hp.counters + 1, sizeof(int32_t), hipMemcpyDeviceToDevice, s));
  }
  return MLPSP_OK;
}

MLPSP_API int mlpsp_render_tilecenter_mfma(const float* rays_o_dev, const float* rays_d_dev,
                                           const void* prim_records_dev, const int32_t* order_dev,
                                           const int32_t* tile_offsets_dev, const float* freq_dev,
                                           const float* att_dev, const void* packed_dev, int num_primitives,
                                           int use_bf16, int width, int height, float threshold, float* out_rgb_dev,
                                           float* out_alpha_dev, int32_t* status_dev, int64_t* counters_dev,
                                           mlpsp_stream_t stream) {
  return mlpsp_render_tilecenter_mfma_feat(rays_o_dev, rays_d_dev, prim_records_dev, order_dev, tile_offsets_dev, 0,
                                           freq_dev, att_dev, packed_dev, num_primitives, use_bf16, nullptr, 0, 0, 0.f,
                                           0.f, width, height, threshold, nullptr, 0, out_rgb_dev, out_alpha_dev,
                                           nullptr, status_dev, counters_dev, 0, nullptr, stream);
}

MLPSP_API int64_t mlpsp_probe_mfma_bf16(int iterations, float* sink_dev, mlpsp_stream_t stream) {
  if (iterations <= 0 || !sink_dev) return -1;
  const int blocks = 256 * 8;      // 8 workgroups of 4 wavefronts per CU: two wavefronts per SIMD
  hipLaunchKernelGGL(probe_mfma_bf16_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, iterations, sink_dev);
  if (hipGetLastError() != hipSuccess) return -1;
  return (int64_t)blocks * 4 * iterations * 8 * (2LL * 32 * 32 * 16);   // FLOPs issued
}

MLPSP_API int mlpsp_probe_issue(const int32_t roles[4], int window_us, void* out_dev, float* sink_dev,
                                mlpsp_stream_t stream) {
  if (!roles || window_us <= 0 || window_us > 100000 || !out_dev || !sink_dev) return MLPSP_E_ARGUMENT;
  for (int k = 0; k < 4; ++k)
    if (roles[k] < 0 || roles[k] > 4) return MLPSP_E_ARGUMENT;
  int rate_khz = 0;
  int dev = 0;
  MLPSP_HIP_TRY(hipGetDevice(&dev));
  MLPSP_HIP_TRY(hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, dev));
  if (rate_khz <= 0) return MLPSP_E_RUNTIME;
  const unsigned long long ticks = (unsigned long long)rate_khz * (unsigned long long)window_us / 1000ull;
  MLPSP_HIP_TRY(hipFuncSetAttribute((const void*)probe_issue_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
  hipLaunchKernelGGL(probe_issue_kernel, dim3(256), dim3(1024), 100 * 1024, (hipStream_t)stream, roles[0], roles[1],
                     roles[2], roles[3], ticks, (ProbeOut*)out_dev, sink_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
