// libmlpsp_hip: the per-tile key + stable sort + conservative culling of one tile, as a device function shared by
// the sort kernel (kept apart from it so that other tile kernels can sort a tile with their own workgroup).
#pragma once
#include "mlpsp_device.hpp"

namespace mlpsp {

// ---------------------------------------------------------------------------------------------
// per-tile key + stable sort.  One 256-thread workgroup per tile.  Each candidate becomes the
// 64-bit word (key bits << 32 | list index): keys are positive floats, whose bit patterns order
// like their values, and the list index in the low word makes equal keys keep list order, which
// is what a stable radix sort on the key alone yields.  The words are ordered in LDS: normally by a
// counting pass into 256 key buckets followed by ranking inside each bucket, else (keys piled up in few
// buckets) by a bitonic network on the next power of two, padded with all-ones words.
//
// Optional conservative culling (cull_threshold in (0,1)): a candidate list comes from a bounding
// circle on screen, and more than half of its entries hit no pixel of the tile -- yet the render
// kernels spend a full 64-lane ray/ellipsoid test on each.  Here, where one LANE handles one
// candidate, the tile's rays are enclosed in the pyramid of its four corner rays (verified against
// every ray of the tile), and a candidate whose threshold ellipsoid {x : (x-c)^T A (x-c) < -2 ln thr}
// lies entirely beyond one of the pyramid's four faces can be hit by no ray of the tile.  For a face
// with inward normal n through the common origin o that is  n.(c-o) < 0  and
// (n.(c-o))^2 >= -2 ln thr * sum_k s_k^2 (R^T n)_k^2, tested with a 2 % margin on the radius, far
// above f32 rounding.  Such an entry is written as ~id (negative) AFTER the tile's sorted survivors, in
// reverse list order: the render kernels skip negative ids, so the image is unchanged bit for bit, and only the
// survivors are ordered.
// ---------------------------------------------------------------------------------------------
constexpr int kSortThreads = 256;
constexpr int kRankPairsMax = 64 * 1024;   // in-bucket comparisons beyond which the sorting network is used instead

// The workgroup's LDS for one tile's sort (27 KB at 2048 entries, 14 KB at 1024).
template <int kSortMax>
struct SortLds {
  // a power of two: the sorting network pads a list to the next power of two inside key[]; a multiple of the
  // workgroup: every thread handles kSortMax / kSortThreads entries; perm[] and order[] hold 16-bit positions
  static_assert((kSortMax & (kSortMax - 1)) == 0 && kSortMax % kSortThreads == 0 && kSortMax <= 65536,
                "capacity of the in-LDS tile sort");
  unsigned long long key[kSortMax];
  int wave_cnt[2][kSortThreads / 64];
  int wave_ok[kSortThreads / 64];
  int cnt[kSortThreads], off[kSortThreads];
  uint16_t perm[kSortMax], order[kSortMax];
  uint32_t kmin, kmax;
  int flags, pairs;
};

// A tile whose list has at most 64 entries, sorted by ONE wavefront (lane = entry) in registers: no LDS, no barrier.
// Same output as sort_one_tile() -- the kept entries ordered by their (key bits, list position) words, which also
// puts keys at or above the invalid key last and in list order among equals; culled entries as ~id at the end of
// the tile's output, last one first -- at a fifth of its instructions: for short lists sort_one_tile()'s cost is
// what four wavefronts spend per tile whatever its length (the pyramid built four times, the passes of the bucket
// ranking, a dozen barriers).  The pyramid and the per-candidate test are those of sort_one_tile(), statement for
// statement.  Requires len <= 64 and len <= capacity; called by a whole wavefront.
__device__ __forceinline__ void sort_small_tile(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ cand, const TileGeom& g, int family, float cull_r2, int num_prims,
    int32_t* __restrict__ sorted_ids, float* __restrict__ sorted_keys, int tile, int start, int n) {
  const int lane = threadIdx.x & 63;
  const int pc = centre_pixel(g, tile);
  const float ox = rays_o[pc * 3 + 0], oy = rays_o[pc * 3 + 1], oz = rays_o[pc * 3 + 2];
  const float dx = rays_d[pc * 3 + 0], dy = rays_d[pc * 3 + 1], dz = rays_d[pc * 3 + 2];
  const int p = (lane < n) ? cand[start + lane] : 0;
  const bool known = (unsigned)p < (unsigned)num_prims;
  const PrimRecord P = prims[known ? p : 0];

  float pox = 0.f, poy = 0.f, poz = 0.f;
  float pn[4][3] = {};
  int faces = 0;
  if (cull_r2 > 0.f) {
    const int tx = tile % g.ntx, ty = tile / g.ntx;
    const int x0 = tx * g.TW, y0 = ty * g.TH;
    const int x1 = min(x0 + g.TW, g.W) - 1, y1 = min(y0 + g.TH, g.H) - 1;
    const int corner[4] = {y0 * g.W + x0, y0 * g.W + x1, y1 * g.W + x1, y1 * g.W + x0};
    float cd[4][3];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int c = 0; c < 3; ++c) cd[j][c] = rays_d[corner[j] * 3 + c];
    pox = rays_o[corner[0] * 3 + 0];
    poy = rays_o[corner[0] * 3 + 1];
    poz = rays_o[corner[0] * 3 + 2];
    int ok = 0x1f;                                       // bits 0..3: face usable; bit 4: common origin
    float nlen[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                        // face j from corner rays j and j+1
      const float* a = cd[j];
      const float* b = cd[(j + 1) & 3];
      const float nx = a[1] * b[2] - a[2] * b[1], ny = a[2] * b[0] - a[0] * b[2], nz = a[0] * b[1] - a[1] * b[0];
      const float side = nx * dx + ny * dy + nz * dz;
      const float len = sqrtf(nx * nx + ny * ny + nz * nz);
      const float sgn = side < 0.f ? -1.f : 1.f;
      pn[j][0] = sgn * nx;
      pn[j][1] = sgn * ny;
      pn[j][2] = sgn * nz;
      nlen[j] = sqrtf(pn[j][0] * pn[j][0] + pn[j][1] * pn[j][1] + pn[j][2] * pn[j][2]);
      if (!(len > 0.f && fabsf(side) > 1e-4f * len)) ok &= ~(1 << j);
    }
    for (int k = lane; k < g.TW * g.TH; k += 64) {
      const int x = x0 + k % g.TW, y = y0 + k / g.TW;
      if (x < g.W && y < g.H) {
        const int pix = y * g.W + x;
        if (rays_o[pix * 3] != pox || rays_o[pix * 3 + 1] != poy || rays_o[pix * 3 + 2] != poz) ok &= ~0x10;
        const float rx = rays_d[pix * 3], ry = rays_d[pix * 3 + 1], rz = rays_d[pix * 3 + 2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float inside = pn[j][0] * rx + pn[j][1] * ry + pn[j][2] * rz;
          if (!(inside >= -1e-6f * nlen[j])) ok &= ~(1 << j);
        }
      }
    }
    int all_ok = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b) all_ok |= __ballot(!((ok >> b) & 1)) ? 0 : (1 << b);
    faces = (all_ok & 0x10) ? (all_ok & 0xf) : 0;
  }

  bool keep = false;
  float key = 0.f;
  if (lane < n) {
    bool outside = false;
    if (faces && known) {
      const float ex = P.cx - pox, ey = P.cy - poy, ez = P.cz - poz;
      const float qw = P.qw, qx = -P.qx, qy = -P.qy, qz = -P.qz;       // conjugate: world -> local
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float nx = pn[j][0], ny = pn[j][1], nz = pn[j][2];
        const float dist = fmaf(nx, ex, fmaf(ny, ey, nz * ez));
        const float tx = 2.f * fmaf(qy, nz, -(qz * ny)), ty = 2.f * fmaf(qz, nx, -(qx * nz)),
                    tz = 2.f * fmaf(qx, ny, -(qy * nx));
        const float lx = fmaf(qw, tx, nx) + fmaf(qy, tz, -(qz * ty));
        const float ly = fmaf(qw, ty, ny) + fmaf(qz, tx, -(qx * tz));
        const float lz = fmaf(qw, tz, nz) + fmaf(qx, ty, -(qy * tx));
        const float h2 = fmaf(P.s2x, lx * lx, fmaf(P.s2y, ly * ly, P.s2z * (lz * lz)));
        outside |= ((faces >> j) & 1) && (dist < 0.f) && (dist * dist >= cull_r2 * h2);
      }
    }
    keep = !outside;
    if (keep)
      key = !known ? kInvalidKey
                   : (family == MLPSP_KEY_DEPTH) ? key_depth(ox, oy, oz, dx, dy, dz, P) : key_tstar(ox, oy, oz, dx, dy, dz, P);
  }
  const uint32_t kb = float_to_bits(key);
  const unsigned long long kept = __ballot(keep);
  int rank = 0;                                          // kept words below this lane's
  for (unsigned long long m = kept; m != 0ull; m &= m - 1ull) {
    const int j = (int)__builtin_ctzll(m);
    const uint32_t kj = (uint32_t)__builtin_amdgcn_readlane((int)kb, j);
    rank += (kj < kb || (kj == kb && j < lane)) ? 1 : 0;
  }
  if (keep) {
    sorted_ids[start + rank] = p;
    if (sorted_keys) sorted_keys[start + rank] = key;
  } else if (lane < n) {
    const unsigned long long culled_before = ~kept & ((1ull << lane) - 1ull);
    const int pos = start + n - 1 - __popcll(culled_before);
    sorted_ids[pos] = ~p;
    if (sorted_keys) sorted_keys[pos] = kInvalidKey;
  }
}

// Sorts one tile with the calling 256-thread workgroup (every thread must call it; `tile` is uniform).  kSortMax
// bounds `capacity`.  A workgroup that sorts several tiles in a row, or uses `lds` for something else afterwards,
// puts a barrier in between.
template <int kSortMax>
__device__ __forceinline__ void sort_one_tile(SortLds<kSortMax>& lds,
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const int32_t* __restrict__ cand, const int32_t* __restrict__ offsets, const TileGeom& g, int family, int capacity,
    float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids, float* __restrict__ sorted_keys, int tile) {
  auto& s_key = lds.key;
  auto& s_wave_cnt = lds.wave_cnt;
  auto& s_wave_ok = lds.wave_ok;
  auto& s_cnt = lds.cnt;
  auto& s_off = lds.off;
  auto& s_perm = lds.perm;
  auto& s_order = lds.order;
  auto& s_kmin = lds.kmin;
  auto& s_kmax = lds.kmax;
  auto& s_flags = lds.flags;
  auto& s_pairs = lds.pairs;
  const int tid = threadIdx.x;
  const int start = offsets[tile];
  const int len = offsets[tile + 1] - start;
  if (len <= 0) return;
  const int n = len < capacity ? len : capacity;

  const int pc = centre_pixel(g, tile);
  const float ox = rays_o[pc * 3 + 0], oy = rays_o[pc * 3 + 1], oz = rays_o[pc * 3 + 2];
  const float dx = rays_d[pc * 3 + 0], dy = rays_d[pc * 3 + 1], dz = rays_d[pc * 3 + 2];

  // Every candidate id this thread will handle is requested up front (at most kSortMax / kSortThreads of them),
  // and the first round's geometry record right behind: their latencies overlap the pyramid phase below, and each
  // round of the key loop then requests the next round's record.
  // An id outside [0, num_prims) (lists that were never validated) reads record 0, is never culled and sorts last
  // with the invalid key; it is passed on unchanged, and the render kernels skip it.
  constexpr int kRounds = kSortMax / kSortThreads;
  int my_id[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) my_id[r] = (tid + r * kSortThreads < n) ? cand[start + tid + r * kSortThreads] : 0;
  PrimRecord P_buf[2];                                   // this round's record and the next round's
  P_buf[0] = prims[((unsigned)my_id[0] < (unsigned)num_prims) ? my_id[0] : 0];

  // ---- the tile's ray pyramid (only when culling is requested).  Every thread builds the four faces from the
  //      corner rays for itself (uniform addresses: one broadcast load each), threads then check the tile's rays
  //      against them, and one barrier combines the verdicts.
  const bool culling = cull_r2 > 0.f;
  const int wave = tid >> 6, lane = tid & 63;
  float pox = 0.f, poy = 0.f, poz = 0.f;
  float pn[4][3] = {};
  int faces = 0;
  if (culling) {
    const int tx = tile % g.ntx, ty = tile / g.ntx;
    const int x0 = tx * g.TW, y0 = ty * g.TH;
    const int x1 = min(x0 + g.TW, g.W) - 1, y1 = min(y0 + g.TH, g.H) - 1;
    const int corner[4] = {y0 * g.W + x0, y0 * g.W + x1, y1 * g.W + x1, y1 * g.W + x0};
    float cd[4][3];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int c = 0; c < 3; ++c) cd[j][c] = rays_d[corner[j] * 3 + c];
    pox = rays_o[corner[0] * 3 + 0];
    poy = rays_o[corner[0] * 3 + 1];
    poz = rays_o[corner[0] * 3 + 2];
    int ok = 0x1f;                                       // bits 0..3: face usable; bit 4: common origin
    float nlen[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                        // face j from corner rays j and j+1
      const float* a = cd[j];
      const float* b = cd[(j + 1) & 3];
      const float nx = a[1] * b[2] - a[2] * b[1], ny = a[2] * b[0] - a[0] * b[2], nz = a[0] * b[1] - a[1] * b[0];
      // orient towards the tile-centre ray; a face the centre ray (nearly) lies in is not used
      const float side = nx * dx + ny * dy + nz * dz;
      const float len = sqrtf(nx * nx + ny * ny + nz * nz);
      const float sgn = side < 0.f ? -1.f : 1.f;
      pn[j][0] = sgn * nx;
      pn[j][1] = sgn * ny;
      pn[j][2] = sgn * nz;
      nlen[j] = sqrtf(pn[j][0] * pn[j][0] + pn[j][1] * pn[j][1] + pn[j][2] * pn[j][2]);
      if (!(len > 0.f && fabsf(side) > 1e-4f * len)) ok &= ~(1 << j);
    }
    // every ray of the tile must start at the common origin and lie inside every face used
    for (int k = tid; k < g.TW * g.TH; k += kSortThreads) {
      const int x = x0 + k % g.TW, y = y0 + k / g.TW;
      if (x < g.W && y < g.H) {
        const int pix = y * g.W + x;
        if (rays_o[pix * 3] != pox || rays_o[pix * 3 + 1] != poy || rays_o[pix * 3 + 2] != poz) ok &= ~0x10;
        const float rx = rays_d[pix * 3], ry = rays_d[pix * 3 + 1], rz = rays_d[pix * 3 + 2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float inside = pn[j][0] * rx + pn[j][1] * ry + pn[j][2] * rz;
          if (!(inside >= -1e-6f * nlen[j])) ok &= ~(1 << j);
        }
      }
    }
    int wave_ok = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b) wave_ok |= __ballot(!((ok >> b) & 1)) ? 0 : (1 << b);
    if (lane == 0) s_wave_ok[wave] = wave_ok;
    __syncthreads();
    ok = s_wave_ok[0];
#pragma unroll
    for (int v = 1; v < kSortThreads / 64; ++v) ok &= s_wave_ok[v];
    faces = (ok & 0x10) ? (ok & 0xf) : 0;
  }

  // ---- keys.  Survivors with an ordinary key are compacted to the front of s_key in list order; survivors
  //      whose key is the invalid key or larger go to the back of s_key, last slot first (the "late" stream: all
  //      of them normally carry the invalid key, and a stable sort leaves those in list order after everything
  //      else); culled entries are written straight to the end of the tile's output, last one first.
  const uint32_t invalid_bits = float_to_bits(kInvalidKey);
  if (tid == 0) {
    s_kmin = 0xffffffffu;
    s_kmax = 0u;
    s_flags = 0;
    s_pairs = 0;
  }
  int nv = 0, nl = 0;                                    // ordinary and late survivors so far (block-uniform)
  uint32_t key_lo = 0xffffffffu, key_hi = 0u;
  bool odd_late = false;
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    if (r * kSortThreads >= n) break;
    const int round = r & 1;
    const int i = r * kSortThreads + tid;
    bool keep = false, outside = false;
    float key = 0.f;
    const PrimRecord& P = P_buf[r & 1];
    const int p = my_id[r];
    if (r + 1 < kRounds && i + kSortThreads < n)
      P_buf[(r + 1) & 1] = prims[((unsigned)my_id[r + 1] < (unsigned)num_prims) ? my_id[r + 1] : 0];
    const bool known = (unsigned)p < (unsigned)num_prims;
    if (i < n) {
      if (faces && known) {
        // (fused multiply-adds here: the test is conservative by a 2 % margin, its roundings are free)
        const float ex = P.cx - pox, ey = P.cy - poy, ez = P.cz - poz;
        const float qw = P.qw, qx = -P.qx, qy = -P.qy, qz = -P.qz;       // conjugate: world -> local
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float nx = pn[j][0], ny = pn[j][1], nz = pn[j][2];
          const float dist = fmaf(nx, ex, fmaf(ny, ey, nz * ez));
          // R^T n = n + qw t + q x t with t = 2 q x n
          const float tx = 2.f * fmaf(qy, nz, -(qz * ny)), ty = 2.f * fmaf(qz, nx, -(qx * nz)),
                      tz = 2.f * fmaf(qx, ny, -(qy * nx));
          const float lx = fmaf(qw, tx, nx) + fmaf(qy, tz, -(qz * ty));
          const float ly = fmaf(qw, ty, ny) + fmaf(qz, tx, -(qx * tz));
          const float lz = fmaf(qw, tz, nz) + fmaf(qx, ty, -(qy * tx));
          const float h2 = fmaf(P.s2x, lx * lx, fmaf(P.s2y, ly * ly, P.s2z * (lz * lz)));
          outside |= ((faces >> j) & 1) && (dist < 0.f) && (dist * dist >= cull_r2 * h2);
        }
      }
      keep = !outside;
      if (keep)
        key = !known ? kInvalidKey
                     : (family == MLPSP_KEY_DEPTH) ? key_depth(ox, oy, oz, dx, dy, dz, P) : key_tstar(ox, oy, oz, dx, dy, dz, P);
    }
    const uint32_t kb = float_to_bits(key);
    const bool late = keep && kb >= invalid_bits;
    const bool front = keep && !late;
    const unsigned long long mf = __ballot(front), ml = __ballot(late);
    if (lane == 0) s_wave_cnt[round][wave] = __popcll(mf) | (__popcll(ml) << 16);
    __syncthreads();                                     // (the two count buffers alternate: one barrier per round)
    int before_f = 0, before_l = 0, total_f = 0, total_l = 0;
#pragma unroll
    for (int v = 0; v < kSortThreads / 64; ++v) {
      const int c = s_wave_cnt[round][v];
      before_f += (v < wave) ? (c & 0xffff) : 0;
      before_l += (v < wave) ? (c >> 16) : 0;
      total_f += c & 0xffff;
      total_l += c >> 16;
    }
    const unsigned long long below = (1ull << lane) - 1ull;
    const int f_before = nv + before_f + __popcll(mf & below);
    const int l_before = nl + before_l + __popcll(ml & below);
    const unsigned long long entry = ((unsigned long long)kb << 32) | (unsigned)i;
    if (front) {
      s_key[f_before] = entry;
    } else if (late) {
      s_key[kSortMax - 1 - l_before] = entry;
    } else if (i < n) {
      const int pos = start + n - 1 - (i - (f_before + l_before));
      sorted_ids[pos] = ~p;
      if (sorted_keys) sorted_keys[pos] = kInvalidKey;
    }
    // range of the ordinary keys (per lane here, combined after the loop), and whether any late key is not the
    // invalid key itself
    key_lo = front ? min(key_lo, kb) : key_lo;
    key_hi = front ? max(key_hi, kb) : key_hi;
    odd_late |= late && kb != invalid_bits;
    nv += total_f;
    nl += total_l;
  }
  {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      key_lo = min(key_lo, (uint32_t)__shfl_xor((int)key_lo, d));
      key_hi = max(key_hi, (uint32_t)__shfl_xor((int)key_hi, d));
    }
    if (lane == 0) {                                     // one pair of LDS atomics per wavefront
      atomicMin(&s_kmin, key_lo);
      atomicMax(&s_kmax, key_hi);
    }
    if (__ballot(odd_late) && lane == 0) atomicOr(&s_flags, 1);
  }
  __syncthreads();

  // ---- order of the ordinary survivors.  Usual case: a counting pass into 256 buckets that are linear in the
  //      key bits between the smallest and the largest key (monotone, so bucket order is key order), then every
  //      entry ranks itself among the entries of its own bucket by its (key, list position) word.  The work of
  //      that last step is the sum of the squared bucket sizes; when keys pile up in few buckets (or a late key
  //      is not the invalid key, which the late stream's list order would misplace) the bitonic network below
  //      sorts instead.
  const uint32_t kmin = s_kmin;
  const float bucket_scale = (float)kSortThreads / ((float)(s_kmax - kmin) + 1.f);
  auto bucket_of = [&](unsigned long long w) {
    const int b = (int)((float)((uint32_t)(w >> 32) - kmin) * bucket_scale);
    return b < kSortThreads - 1 ? b : kSortThreads - 1;
  };
  bool network = (s_flags & 1) != 0;
  const bool ranked = !network && nv > 1;
  if (ranked) {
    s_cnt[tid] = 0;
    __syncthreads();
    for (int i = tid; i < nv; i += kSortThreads) atomicAdd(&s_cnt[bucket_of(s_key[i])], 1);
    __syncthreads();
    const int c = s_cnt[tid];
    int incl = c, pairs = c * c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) pairs += __shfl_xor(pairs, d);
    if (lane == 63) s_wave_cnt[0][wave] = incl;
    if (lane == 0) atomicAdd(&s_pairs, pairs);
    __syncthreads();
    int base = 0;
#pragma unroll
    for (int v = 0; v < kSortThreads / 64; ++v) base += (v < wave) ? s_wave_cnt[0][v] : 0;
    const int excl = base + incl - c;
    s_off[tid] = excl;
    s_cnt[tid] = excl;                                   // from here on: the bucket's fill cursor
    network = s_pairs > kRankPairsMax;
    __syncthreads();
    if (!network) {
      for (int i = tid; i < nv; i += kSortThreads) s_perm[atomicAdd(&s_cnt[bucket_of(s_key[i])], 1)] = (uint16_t)i;
      __syncthreads();
      for (int a = tid; a < nv; a += kSortThreads) {
        const int ia = s_perm[a];
        const unsigned long long wa = s_key[ia];
        const int b = bucket_of(wa);
        const int lo = s_off[b], hi = s_cnt[b];          // the cursor ended at the bucket's end
        int r = 0;
        for (int q = lo; q < hi; ++q) r += (s_key[s_perm[q]] < wa) ? 1 : 0;
        s_order[lo + r] = (uint16_t)ia;
      }
    }
  }
  if (network) {
    // the late entries join the others (through registers: the two regions can overlap)
    unsigned long long moved[kSortMax / kSortThreads];
#pragma unroll
    for (int v = 0; v < kSortMax / kSortThreads; ++v) {
      const int j = tid + v * kSortThreads;
      moved[v] = (j < nl) ? s_key[kSortMax - 1 - j] : 0ull;
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < kSortMax / kSortThreads; ++v) {
      const int j = tid + v * kSortThreads;
      if (j < nl) s_key[nv + j] = moved[v];
    }
    nv += nl;
    nl = 0;
    int npad = 2;
    while (npad < nv) npad <<= 1;
    for (int i = nv + tid; i < npad; i += kSortThreads) s_key[i] = ~0ull;
    __syncthreads();

    // Bitonic network.  Thread t of a step handles the pair (lo, lo | j) with lo built from t, so for
    // j < 64 the 64 lanes of a wavefront touch only their own 128 consecutive entries: those steps
    // need no workgroup barrier, only program order inside the wavefront (LDS operations of one
    // wavefront complete in order).  A workgroup barrier separates any step with j >= 64 from its
    // neighbours.
    int prev_j = 64;
    for (int k = 2; k <= npad; k <<= 1) {
      for (int j = k >> 1; j > 0; j >>= 1) {
        if (j >= 64 || prev_j >= 64) __syncthreads();
        else {
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
        prev_j = j;
        for (int t = tid; t < (npad >> 1); t += kSortThreads) {
          const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1));
          const int hi = lo | j;
          const unsigned long long a = s_key[lo], b = s_key[hi];
          const bool ascending = (lo & k) == 0;
          if ((a > b) == ascending) {
            s_key[lo] = b;
            s_key[hi] = a;
          }
        }
      }
    }
  }
  __syncthreads();

  const bool through_order = ranked && !network;
  for (int i = tid; i < len; i += kSortThreads) {
    if (i < nv + nl) {
      const unsigned long long w = (i >= nv) ? s_key[kSortMax - 1 - (i - nv)] : s_key[through_order ? s_order[i] : i];
      sorted_ids[start + i] = cand[start + (int)(w & 0xffffffffu)];
      if (sorted_keys) sorted_keys[start + i] = bits_to_float((uint32_t)(w >> 32));
    } else if (i >= n) {
      sorted_ids[start + i] = cand[start + i];     // beyond the sort capacity: list order, never culled
      if (sorted_keys) sorted_keys[start + i] = kInvalidKey;
    }
  }
}

}  // namespace mlpsp
