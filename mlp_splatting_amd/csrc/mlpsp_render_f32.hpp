// The scalar-f32 tile-centre render kernel (shared by the RGB entry point and the feature entry point,
// which asks it to emit hit records).
#pragma once
#include <cstdlib>
#include "mlpsp_device.hpp"
#include "mlpsp_hitrec.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_mlp.hpp"
#include "mlpsp_mlp_mfma32.hpp"

namespace mlpsp {

// EMIT = 0: image only.  EMIT = 1 / 2: also emit one hit record per primitive that hits a pixel of this
// wavefront, float[K][64] with K = 1 (the compositing weight w) / K = 5 (w and the four tetrahedral
// gates); w = -1 marks a pixel the primitive did not hit (weights are never negative).
//
// STATS: also accumulate the pruning statistics of np_tile_kernels.cu:2139-2519: per processed primitive
// the wavefront reduces over its pixels  w,  max w,  [w > 1e-8],  [w > 0.1] * w * err  and  [w > 0.1]
// (err = L1 colour error of the pixel after this blend step against gt_rgb) and adds them to the five
// per-primitive buffers with atomics, as the reference does per block (:2435-2456).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) v += __shfl_xor(v, d);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) v = fmaxf(v, __shfl_xor(v, d));
  return v;
}

// MF: the 72->32->32->4 MLP runs on the matrix cores for all 64 pixels at once (mlp_wave_mfma32, same bits);
// requires HT == 32 or 16, FT == 6 and 16-byte aligned weight arrays.
template <int HT, int FT, int EMIT, bool STATS = false, bool MF = false>
__global__ __launch_bounds__(64) void render_tilecenter_f32_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, int F, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ W2, const float* __restrict__ b2, const float* __restrict__ W3,
    const float* __restrict__ b3, int N, int H, TileGeom g, int waves_per_tile, int per_xcd,
    int num_items, float thr, float* __restrict__ out_rgb, float* __restrict__ out_alpha, float* __restrict__ out_t,
    unsigned long long* __restrict__ counters, float beta, float temp, HitPool hp,
    const float* __restrict__ gt_rgb = nullptr, float* __restrict__ stat_sum_w = nullptr,
    float* __restrict__ stat_max_w = nullptr, int32_t* __restrict__ stat_hits = nullptr,
    float* __restrict__ stat_sum_werr = nullptr, int32_t* __restrict__ stat_contrib = nullptr) {
  // The weight pointers are separate __restrict__ parameters (not a struct): only then does the compiler
  // know that the record stores below cannot alias them and keeps fetching weights with scalar loads.
  const MlpPtrs mlp{W1, b1, W2, b2, W3, b3};
  // XCD-aware work assignment: XCD k (blockIdx.x % 8) walks items [k*per_xcd, (k+1)*per_xcd).
  const int item = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (item >= num_items) return;
  const int tile = item / waves_per_tile, wslot = item % waves_per_tile;
  const int slot = wslot * 64 + threadIdx.x;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int lx = slot % g.TW, ly = slot / g.TW;
  const int x = tx * g.TW + lx, y = ty * g.TH + ly;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;

  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f;
  const float roy = valid ? rays_o[pix * 3 + 1] : 0.f;
  const float roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f;
  const float rdy = valid ? rays_d[pix * 3 + 1] : 0.f;
  const float rdz = valid ? rays_d[pix * 3 + 2] : 0.f;

  const int start = offsets[tile];
  const int end = offsets[tile + 1];

  PixelAcc acc = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
  unsigned n_proc = 0, n_proc_hit = 0, n_hits = 0;
  float gtr = 0.f, gtg = 0.f, gtb = 0.f;
  if constexpr (STATS) {
    if (valid) {
      gtr = gt_rgb[pix * 3 + 0];
      gtg = gt_rgb[pix * 3 + 1];
      gtb = gt_rgb[pix * 3 + 2];
    }
  }
  HitEmitter em = hit_emitter_begin(hp, wslot, start, tile);
  DirOperands dir;
  if constexpr (MF) encode_direction(rdx, rdy, rdz, freq, att, dir);

  for (int i = start; i < end; ++i) {
    const int p = __builtin_amdgcn_readfirstlane(order[i]);
    if (p < 0 || p >= N) continue;
    const PrimRecord P = prims[p];
    HitInfo h;
    const bool live = valid && (acc.trans >= kTransmittanceFloor);
    const bool hit = live && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
    const unsigned long long hit_mask = __ballot(hit);
    ++n_proc;
    if (hit_mask != 0ull) {
      ++n_proc_hit;
      n_hits += __popcll(hit_mask);
      int rs = -1;
      float w_stat = 0.f;
      if constexpr (EMIT > 0) rs = hit_emitter_next(hp, em, (int)threadIdx.x);
      float* __restrict__ rec = reinterpret_cast<float*>(hp.records + (size_t)(rs < 0 ? 0 : rs) * hp.record_bytes);
      // (lanes that did not hit carry no hit point; the matrix-core evaluation runs on all 64 lanes)
      const float x6[6] = {rdx, rdy, rdz, hit ? h.dx : 0.f, hit ? h.dy : 0.f, hit ? h.dz : 0.f};
      float o[4];
      if constexpr (MF) mlp_wave_mfma32<false, false, HT>(x6, freq, att, W1, b1, W2, b2, W3, b3, p, dir, o);
      if (hit) {
        if constexpr (!MF) mlp_eval<HT, FT>(x6, freq, att, F, H, mlp, p, o);
        const float w = blend_step(acc, o[0], o[1], o[2], o[3], h.decay, h.t);
        w_stat = w;
        if constexpr (EMIT > 0) {
          if (rs >= 0) {
            rec[threadIdx.x] = w;
            if constexpr (EMIT > 1) {
              float gt[4];
              tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gt);
#pragma unroll
              for (int k = 0; k < 4; ++k) rec[(k + 1) * 64 + threadIdx.x] = gt[k];
            }
          }
        }
      } else if constexpr (EMIT > 0) {
        if (rs >= 0) rec[threadIdx.x] = -1.f;       // the gates of a missed pixel are never read
      }
      if constexpr (EMIT > 0) {
        if (rs >= 0 && threadIdx.x == 0) hp.hit_ids[rs] = p;
      }
      if constexpr (STATS) {
        const float lw = hit ? w_stat : 0.f;
        const bool contrib = hit && (lw > 1e-1f);
        float lerr = 0.f;
        if (contrib) lerr = lw * ((fabsf(acc.cr - gtr) + fabsf(acc.cg - gtg)) + fabsf(acc.cb - gtb));
        const float s_w = wave_sum(lw), m_w = wave_max(lw), s_err = wave_sum(lerr);
        const int n_hit = __popcll(__ballot(hit && (lw > 1e-8f))), n_con = __popcll(__ballot(contrib));
        if (threadIdx.x == 0) {
          atomicAdd(stat_sum_w + p, s_w);
          atomicMax(reinterpret_cast<int*>(stat_max_w + p), __float_as_int(m_w));   // weights are >= 0
          atomicAdd(stat_hits + p, n_hit);
          if (stat_sum_werr) atomicAdd(stat_sum_werr + p, s_err);
          if (stat_contrib) atomicAdd(stat_contrib + p, n_con);
        }
      }
    }
    if (__ballot(valid && (acc.trans >= kTransmittanceFloor)) == 0ull) break;
  }

  if (valid) {
    out_rgb[pix * 3 + 0] = acc.cr;
    out_rgb[pix * 3 + 1] = acc.cg;
    out_rgb[pix * 3 + 2] = acc.cb;
    out_alpha[pix] = 1.f - acc.trans;
    if (out_t) out_t[pix] = acc.t_acc / (acc.w_acc > 1e-8f ? acc.w_acc : 1.f);
  }
  if constexpr (EMIT > 0) {
    if (threadIdx.x == 0) hp.item_hits[item] = em.count;
  }
  if (counters && threadIdx.x == 0) {
    atomicAdd(counters + 1, (unsigned long long)n_proc);
    atomicAdd(counters + 2, (unsigned long long)n_proc_hit);
    atomicAdd(counters + 3, (unsigned long long)n_hits);
  }
}

// The same walk (image only, matrix-core evaluation) for launches too small to fill the chip: a few hundred tiles on
// a thousand SIMDs leave every wavefront alone on its SIMD, where nothing hides the chain id -> geometry record ->
// hit test -> weight rows -> MLP, and the launch lasts as long as its longest tile.  Two things shorten that chain.
// (1) The ids of a tile are read 64 at a time (one per lane), and the NEXT entry's geometry record and layer-1
// operands are requested before the current entry is tested and evaluated, whether or not that entry will hit:
// registers are plentiful when one wavefront has the SIMD to itself.  (Layer 2's operands are requested as an
// evaluation begins: they arrive behind layer 1's instructions.)  (2) HALF: two wavefronts share a 64-pixel item,
// each takes 32 of its pixels -- every pixel on two lanes that carry the same state -- and evaluates one column block,
// half the matrix instructions (mlp_half_mfma32_with).  Pixels are independent (a pixel below the transmittance floor
// never blends again, so a wavefront that stops early stops nothing its pixels would still have done).
// Same arithmetic in the same order either way: same bits.  Work counters are kept per 64-pixel item: the caller
// does not ask for them with HALF.
template <int HT, bool HALF>
__global__ __launch_bounds__(64) void render_tilecenter_f32_ahead_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const float* __restrict__ freq,
    const float* __restrict__ att, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ W2, const float* __restrict__ b2, const float* __restrict__ W3,
    const float* __restrict__ b3, int N, TileGeom g, int waves_per_tile, int per_xcd, int num_items, float thr,
    float* __restrict__ out_rgb, float* __restrict__ out_alpha, float* __restrict__ out_t,
    unsigned long long* __restrict__ counters) {
  // (with HALF, num_items and per_xcd count half items)
  const int unit = (blockIdx.x % kNumXcd) * per_xcd + blockIdx.x / kNumXcd;
  if (unit >= num_items) return;
  const int item = HALF ? unit >> 1 : unit;
  const int tile = item / waves_per_tile, wslot = item % waves_per_tile;
  const int lane = (int)threadIdx.x;
  const int slot = HALF ? wslot * 64 + (unit & 1) * 32 + (lane & 31) : wslot * 64 + lane;
  const bool writer = !HALF || lane < 32;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int lx = slot % g.TW, ly = slot / g.TW;
  const int x = tx * g.TW + lx, y = ty * g.TH + ly;
  const bool valid = (slot < g.TW * g.TH) && (x < g.W) && (y < g.H);
  const int pix = valid ? (y * g.W + x) : 0;
  const float rox = valid ? rays_o[pix * 3 + 0] : 0.f;
  const float roy = valid ? rays_o[pix * 3 + 1] : 0.f;
  const float roz = valid ? rays_o[pix * 3 + 2] : 0.f;
  const float rdx = valid ? rays_d[pix * 3 + 0] : 0.f;
  const float rdy = valid ? rays_d[pix * 3 + 1] : 0.f;
  const float rdz = valid ? rays_d[pix * 3 + 2] : 0.f;
  const int start = offsets[tile];
  const int end = offsets[tile + 1];

  PixelAcc acc = {0.f, 0.f, 0.f, 1.f, 0.f, 0.f};
  unsigned n_proc = 0, n_proc_hit = 0, n_hits = 0;
  DirOperands dir;
  float dir_half[18];
  if constexpr (HALF) encode_direction_half(rdx, rdy, rdz, freq, att, dir_half);
  else encode_direction(rdx, rdy, rdz, freq, att, dir);

  bool done = false;
  for (int base = start; base < end && !done; base += 64) {
    const int n = min(64, end - base);
    const int idv = lane < n ? order[base + lane] : -1;
    // entry 0 of this stretch: nothing to hide its requests behind
    int p = __builtin_amdgcn_readlane(idv, 0);
    bool ok = p >= 0 && p < N;
    PrimRecord P = prims[ok ? p : 0];
    MlpLayer1<HT> w;
    request_layer1<HT>(W1, b1, ok ? p : 0, w);
    for (int k = 0; k < n; ++k) {
      // the next entry's record and operands, under way while this one is worked on (an id outside [0, N) and the
      // entry after the last one request primitive 0 and are not used)
      const int q = __builtin_amdgcn_readlane(idv, min(k + 1, 63));
      const bool ok_next = k + 1 < n && q >= 0 && q < N;
      const int p_next = ok_next ? q : 0;
      const PrimRecord P_next = prims[p_next];
      MlpLayer1<HT> w_next;
      request_layer1<HT>(W1, b1, p_next, w_next);
      if (ok) {
        HitInfo h;
        const bool live = valid && (acc.trans >= kTransmittanceFloor);
        const bool hit = live && hit_rot(rox, roy, roz, rdx, rdy, rdz, P, thr, h);
        const unsigned long long hit_mask = __ballot(hit);
        ++n_proc;
        if (hit_mask != 0ull) {
          ++n_proc_hit;
          n_hits += __popcll(hit_mask);
          // (lanes that did not hit carry no hit point; the matrix-core evaluation runs on all 64 lanes)
          const float x6[6] = {rdx, rdy, rdz, hit ? h.dx : 0.f, hit ? h.dy : 0.f, hit ? h.dz : 0.f};
          float o[4];
          MlpLayer2<HT> w2;
          request_layer2<HT>(W2, b2, p, w2);
          if constexpr (HALF) mlp_half_mfma32_with<HT>(w, w2, x6, freq, att, W3, b3, p, dir_half, o);
          else mlp_wave_mfma32_with<false, false, HT>(w, w2, x6, freq, att, W3, b3, p, dir, o);
          if (hit) blend_step(acc, o[0], o[1], o[2], o[3], h.decay, h.t);
        }
        if (__ballot(valid && (acc.trans >= kTransmittanceFloor)) == 0ull) {
          done = true;
          break;
        }
      }
      p = p_next;
      ok = ok_next;
      P = P_next;
      w = w_next;
    }
  }

  if (valid && writer) {
    out_rgb[pix * 3 + 0] = acc.cr;
    out_rgb[pix * 3 + 1] = acc.cg;
    out_rgb[pix * 3 + 2] = acc.cb;
    out_alpha[pix] = 1.f - acc.trans;
    if (out_t) out_t[pix] = acc.t_acc / (acc.w_acc > 1e-8f ? acc.w_acc : 1.f);
  }
  if (!HALF && counters && lane == 0) {
    atomicAdd(counters + 1, (unsigned long long)n_proc);
    atomicAdd(counters + 2, (unsigned long long)n_proc_hit);
    atomicAdd(counters + 3, (unsigned long long)n_hits);
  }
}

// Which of the two kernels above a launch of `items` 64-pixel items takes: 2 = two wavefronts per item (at most one
// wavefront per SIMD of the chip's 1,024, and no work counters asked for), 1 = one wavefront per item with the next
// entry requested ahead (at most 1,024 items), 0 = neither (the kernel for launches that fill the chip).
// MLPSP_F32_AHEAD=0 / 1 / 2 in the environment overrides the size rule (comparison runs, tests); 2 still needs a
// launch without counters.
constexpr int kAheadItems = 1024;
inline int ahead_mode(int64_t items, int num_primitives, bool counters) {
  if (num_primitives <= 0) return 0;
  int mode = items * 2 <= kAheadItems ? 2 : items <= kAheadItems ? 1 : 0;
  const char* e = getenv("MLPSP_F32_AHEAD");
  if (e && e[0] >= '0' && e[0] <= '2' && items * 2 <= 2147483647LL - 8) mode = e[0] - '0';
  return (mode == 2 && counters) ? 1 : mode;
}

// Whether the matrix-core f32 evaluation applies: the 72->32->32->4 or 72->16->16->4 shape, weight arrays that can be
// read 16 bytes at a time, and no request for the scalar kernel (environment MLPSP_F32_SCALAR=1, which
// exists for comparison runs).
inline bool use_mfma32(int hidden, int num_frequencies, const float* W1, const float* b1, const float* W2,
                       const float* b2) {
  if ((hidden != 32 && hidden != 16) || num_frequencies != 6) return false;
  if (((uintptr_t)W1 | (uintptr_t)b1 | (uintptr_t)W2 | (uintptr_t)b2) & 15u) return false;
  const char* e = getenv("MLPSP_F32_SCALAR");
  return !(e && e[0] == '1');
}

}  // namespace mlpsp

