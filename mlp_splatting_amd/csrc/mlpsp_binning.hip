// libmlpsp_hip: projection of primitive supports and tile binning (the "legacy" screen-space rule).
//
// The reference evaluates a dense [tiles x primitives] boolean matrix (scannet/cumodel.py:1028-1070).
// Here the same predicate is evaluated sparsely and deterministically, without atomics on global
// memory and without a sort, in two levels:
//   level 1: the frame is cut into super-tiles of 8x8 tiles.  Wavefront (chunk c, super-tile s)
//            tests 2048 consecutive primitives against the super-tile rectangle (a superset of the
//            union of its tiles' tests) and counts; the fill pass writes the survivors in ascending
//            id order -> one ascending candidate list per super-tile.  With one view and a screen of
//            few super-tiles the counting goes the other way round: every primitive finds the
//            super-tiles it overlaps (bin_level1_scatter_kernel, which also computes the bounds).
//   level 2: one wavefront per tile walks its super-tile's list 64 ids at a time, applies the exact
//            per-tile test and counts with a ballot; the fill pass writes the tile's candidates at
//            ballot-prefix positions -> tile-major lists, ascending id inside a tile, which is the
//            order `nonzero()` on the dense matrix yields.
// A fill pass needs the exclusive prefix sums of the counts.  Its workgroups form their own from the
// counts (level 1) or from per-workgroup sums the counting pass leaves (level 2): four launches per
// frame, count and fill of each level.  Only the two-call interface, whose caller sizes the candidate
// buffer between the calls, scans the tile counts with a kernel of its own.
// All kernels are HBM/L2-bound integer and compare work; nothing here wants MFMA.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"

#include <math.h>
#include <stdlib.h>

namespace mlpsp {

constexpr int kSuper = 8;       // tiles per super-tile side
constexpr int kChunk = 2048;    // primitives per level-1 workgroup
constexpr int kBinThreads = 256;
constexpr int kWideThreads = 1024;              // workgroups that work out their own place in a list of lists
constexpr int kL2Group = kWideThreads / 64;     // tiles per level-2 workgroup

// what the level-2 counting pass leaves per workgroup, so that the fill pass can place its tiles without a scan
// kernel in between
struct L2Group {
  long long sum;      // entries of the group's tile lists
  int longest;        // its longest tile list
  int pad;
};

struct BinScratch {
  float* mats;        // K view matrices (16 floats each) then the projection (16 floats)
  float4* bounds;     // [K][N] (minx, maxx, miny, maxy); all NaN when behind the near plane
  int32_t* l1_counts; // [S*NC + 1] survivors per (super-tile, chunk)
  int32_t* l1_super;  // [S + 1] where each super-tile's list starts in l1_list (clamped to l1_capacity)
  long long* totals;  // [0] level-1 entries, [1] tile-list entries, [2] longest tile list, [3] guard status
  struct L2Group* groups;   // [ceil(T / 16)] entries and longest list of every 16 consecutive tiles
  int32_t* l1_list;   // [l1_capacity]
  float4* l1_bounds;  // [l1_capacity] bounds of the listed primitives under the super-tile's view (garbage for a
                      // super-tile whose tiles use several views: super_view says which)
  int32_t* super_view;    // [S] the one view all tiles of the super-tile use, or -1
  long long l1_capacity;
  // survivor masks of the counting passes (one ballot per 64 tested entries), so that the fill passes neither
  // re-read the bounds nor repeat the tests:
  unsigned long long* l1_masks;   // [S*NC][kChunk/64]
  unsigned long long* l2_masks;   // [64 tiles of a super-tile][l1_capacity/64 + S + 1]
  long long l2_mask_stride;
};

__host__ __device__ inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

inline BinScratch carve(void* base, size_t bytes, int N, int K, int S, int NC) {
  BinScratch b;
  char* p = static_cast<char*>(base);
  size_t off = 0;
  b.mats = reinterpret_cast<float*>(p + off);
  off += align256((size_t)(K + 1) * 16 * sizeof(float));
  b.bounds = reinterpret_cast<float4*>(p + off);
  off += align256((size_t)K * N * sizeof(float4));
  b.l1_counts = reinterpret_cast<int32_t*>(p + off);
  off += align256(((size_t)S * NC + 1) * sizeof(int32_t));
  b.totals = reinterpret_cast<long long*>(p + off);
  off += 256;
  // the level-1 lists carry the bounds next to the ids (20 bytes per entry), so that level 2 streams them
  // instead of gathering 16 bytes per lane from all over the bounds array
  b.l1_masks = reinterpret_cast<unsigned long long*>(p + off);
  off += align256((size_t)S * NC * (kChunk / 64) * sizeof(unsigned long long));
  b.super_view = reinterpret_cast<int32_t*>(p + off);
  off += align256((size_t)S * sizeof(int32_t));
  b.l1_super = reinterpret_cast<int32_t*>(p + off);
  off += align256(((size_t)S + 1) * sizeof(int32_t));
  b.groups = reinterpret_cast<L2Group*>(p + off);           // a super-tile has at most 64 tiles = 4 groups
  off += align256(((size_t)S * (64 / kL2Group) + 1) * sizeof(L2Group));
  // per level-1 entry: 4 bytes id + 16 bytes bounds + 64 mask bits for the 64 tiles = 8 bytes
  const size_t entry = sizeof(int32_t) + sizeof(float4) + 8;
  const size_t fixed = off + 1024 + align256((size_t)(S + 1) * 64 * sizeof(unsigned long long));
  b.l1_capacity = bytes > fixed ? (long long)((bytes - fixed) / entry) : 0;
  b.l1_capacity = (b.l1_capacity < 2147483584LL ? b.l1_capacity : 2147483584LL) & ~63LL;   // positions are 32-bit
  b.l1_list = reinterpret_cast<int32_t*>(p + off);
  off += align256((size_t)b.l1_capacity * sizeof(int32_t));
  b.l1_bounds = reinterpret_cast<float4*>(p + off);
  off += align256((size_t)b.l1_capacity * sizeof(float4));
  b.l2_mask_stride = b.l1_capacity / 64 + S + 1;
  b.l2_masks = reinterpret_cast<unsigned long long*>(p + off);
  return b;
}

struct BinGeom {
  int W, H, ts, ntx, nty, nsx, nsy, N, K, NC;
};

// Screen-space bounds of primitive i under view k (scannet/cumodel.py:1001-1041).  The 4-term dot
// products are fma chains from the last term inwards.
// One view: the two matrices travel as kernel arguments (no host-to-device copy in front of the frame).
struct BinMats {
  float v[16], p[16];
};

// MODE 0: K view matrices then the projection at `mats` (device).  MODE 1: one view, both matrices in `one`.
// MODE 2: one view, the view matrix at `mats` and the projection at `proj_dev` (device tensors of the caller: no
// host copy of them exists, so the focal length is formed here, with the host's expression).
template <int MODE>
__device__ __forceinline__ float4 primitive_bounds(const float* __restrict__ pos, const float* __restrict__ logs,
                                                   const float* __restrict__ mats, const float* __restrict__ proj_dev,
                                                   const BinMats& one, const BinGeom& g, float rm, float focal, int i,
                                                   int k) {
  const float* V = MODE == 1 ? one.v : mats + k * 16;
  const float* Pm = MODE == 1 ? one.p : MODE == 2 ? proj_dev : mats + g.K * 16;
  if (MODE == 2) focal = ((Pm[0] * (float)g.W) / 2.0f + (Pm[5] * (float)g.H) / 2.0f) * 0.5f;
  const float x = pos[i * 3 + 0], y = pos[i * 3 + 1], z = pos[i * 3 + 2];
  float pv[4], clip[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) pv[r] = fmaf(V[r * 4 + 0], x, fmaf(V[r * 4 + 1], y, fmaf(V[r * 4 + 2], z, V[r * 4 + 3])));
  const float depth = pv[2];
  const float s = fmaxf(fmaxf(det_exp(logs[i * 3 + 0]), det_exp(logs[i * 3 + 1])), det_exp(logs[i * 3 + 2]));
  const float world_radius = s * rm;
  const float pr = (world_radius / (depth + 1e-8f)) * focal;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    clip[r] = fmaf(Pm[r * 4 + 0], pv[0], fmaf(Pm[r * 4 + 1], pv[1], fmaf(Pm[r * 4 + 2], pv[2], Pm[r * 4 + 3] * pv[3])));
  float w = clip[3];
  w = (w == 0.f) ? w + 1e-6f : w;
  const float sx = (((clip[0] / w) + 1.f) * 0.5f) * (float)g.W;
  const float sy = (((clip[1] / w) + 1.f) * 0.5f) * (float)g.H;
  const float nan = __builtin_nanf("");
  const bool front = depth > 0.001f;
  return front ? make_float4(sx - pr, sx + pr, sy - pr, sy + pr) : make_float4(nan, nan, nan, nan);
}

template <int MODE>
__global__ __launch_bounds__(kBinThreads) void bin_bounds_kernel(const float* __restrict__ pos,
                                                                 const float* __restrict__ logs,
                                                                 const float* __restrict__ mats,
                                                                 const float* __restrict__ proj_dev, BinMats one,
                                                                 BinGeom g, float rm, float focal,
                                                                 float4* __restrict__ bounds) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int k = blockIdx.y;
  if (i >= g.N) return;
  bounds[(size_t)k * g.N + i] = primitive_bounds<MODE>(pos, logs, mats, proj_dev, one, g, rm, focal, i, k);
}

// strict inequalities of scannet/cumodel.py:1043-1044 on an axis-aligned pixel rectangle
__device__ __forceinline__ bool rect_overlap(const float4 b, float x0, float x1, float y0, float y1) {
  return (b.x < x1) && (b.y > x0) && (b.z < y1) && (b.w > y0);
}

__device__ __forceinline__ bool super_overlap(const float4* __restrict__ bounds, const BinGeom& g, int i, float x0,
                                              float x1, float y0, float y1) {
  bool any = false;
  for (int k = 0; k < g.K; ++k) any |= rect_overlap(bounds[(size_t)k * g.N + i], x0, x1, y0, y1);
  return any;
}

__device__ __forceinline__ void super_rect(const BinGeom& g, int s, float& x0, float& x1, float& y0, float& y1) {
  const int sx = s % g.nsx, sy = s / g.nsx;
  x0 = (float)(sx * kSuper * g.ts);
  y0 = (float)(sy * kSuper * g.ts);
  x1 = (float)(min((sx + 1) * kSuper, g.ntx) * g.ts);
  y1 = (float)(min((sy + 1) * kSuper, g.nty) * g.ts);
}

// mask `which` (wave-uniform) of the 64-bit values held one per lane
__device__ __forceinline__ unsigned long long lane_value(unsigned long long v, int which) {
  const unsigned lo = __builtin_amdgcn_readlane((unsigned)v, which);
  const unsigned hi = __builtin_amdgcn_readlane((unsigned)(v >> 32), which);
  return ((unsigned long long)hi << 32) | lo;
}

// position of the n-th (from 0) set bit of m; n < popcount(m)
__device__ __forceinline__ int nth_set_bit(unsigned long long m, int n) {
  unsigned x = (unsigned)m;
  int pos = 0, c = __popc(x);
  if (n >= c) {
    n -= c;
    pos = 32;
    x = (unsigned)(m >> 32);
  }
#pragma unroll
  for (int width = 16; width >= 1; width >>= 1) {
    c = __popc(x & ((1u << width) - 1u));
    if (n >= c) {
      n -= c;
      pos += width;
      x >>= width;
    }
  }
  return pos;
}

__device__ __forceinline__ unsigned lanes_below(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

// level 1, counting pass by (chunk, super-tile).  grid = (NC, ceil(S / 4)); wavefront w of a workgroup owns super-tile
// 4 * blockIdx.y + w and walks the chunk's 2048 primitives 64 at a time (no workgroup barrier: counts come from
// ballots, which are kept for the fill pass): l1_counts[s*NC + c] = survivors.
__global__ __launch_bounds__(kBinThreads) void bin_level1_kernel(const float4* __restrict__ bounds, BinGeom g,
                                                                 const int32_t* __restrict__ tile_view_ids,
                                                                 int32_t* __restrict__ l1_counts,
                                                                 unsigned long long* __restrict__ l1_masks,
                                                                 int32_t* __restrict__ super_view) {
  const int c = blockIdx.x, s = blockIdx.y * (kBinThreads / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= g.nsx * g.nsy) return;
  float x0, x1, y0, y1;
  super_rect(g, s, x0, x1, y0, y1);
  // Several views: only the views that tiles of this super-tile actually use can contribute (lane l looks
  // at tile l of the 8 x 8 block); up to four distinct ones are kept, more fall back to testing all K.
  int nviews = g.K, v0 = 0, v1 = 0, v2 = 0, v3 = 0;
  if (g.K > 1 && tile_view_ids) {
    const int tx = (s % g.nsx) * kSuper + (lane & 7), ty = (s / g.nsx) * kSuper + (lane >> 3);
    const bool has = tx < g.ntx && ty < g.nty;
    const int view = has ? tile_view_ids[ty * g.ntx + tx] : -1;
    unsigned long long pending = __ballot(has);
    int found = 0;
    while (pending != 0ull && found <= 4) {
      const int v = __builtin_amdgcn_readlane(view, (int)__builtin_ctzll(pending));
      pending &= ~__ballot(has && view == v);
      if (found == 0) v0 = v;
      else if (found == 1) v1 = v;
      else if (found == 2) v2 = v;
      else if (found == 3) v3 = v;
      ++found;
    }
    if (found <= 4) nviews = -found;       // negative: use the explicit list
  }
  // one view for the whole super-tile (always so with one camera): the fast paths below, here and in level 2
  const bool single = g.K == 1 || nviews == -1;
  const float4* __restrict__ sb = bounds + (size_t)(g.K == 1 ? 0 : v0) * g.N;
  if (c == 0 && lane == 0) super_view[s] = single ? (g.K == 1 ? 0 : v0) : -1;
  long long running = 0;
  const int first = c * kChunk;
  unsigned long long* __restrict__ masks = l1_masks + ((size_t)s * g.NC + c) * (kChunk / 64);
  static_assert(kChunk / 64 <= 64, "one ballot per lane");
  unsigned long long mine = 0ull;
  if (single) {
    // one view: eight independent 16-byte loads in flight per step (NaN bounds fail every comparison)
    const float nanv = __builtin_nanf("");
    for (int r0 = 0; r0 < kChunk / 64; r0 += 8) {
      float4 bb[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = first + (r0 + u) * 64 + lane;
        bb[u] = (i < g.N) ? sb[i] : make_float4(nanv, nanv, nanv, nanv);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const unsigned long long m = __ballot(rect_overlap(bb[u], x0, x1, y0, y1));
        mine = (lane == r0 + u) ? m : mine;
        running += __popcll(m);
      }
    }
    if (lane < kChunk / 64) masks[lane] = mine;
    if (lane == 0) l1_counts[s * g.NC + c] = (int32_t)running;
    return;
  }
#pragma unroll 4
  for (int r = 0; r < kChunk / 64; ++r) {
    const int i = first + r * 64 + lane;
    bool keep = false;
    if (i < g.N) {
      if (nviews >= 0) {
        keep = super_overlap(bounds, g, i, x0, x1, y0, y1);
      } else {
        keep = rect_overlap(bounds[(size_t)v0 * g.N + i], x0, x1, y0, y1);
        if (nviews <= -2) keep |= rect_overlap(bounds[(size_t)v1 * g.N + i], x0, x1, y0, y1);
        if (nviews <= -3) keep |= rect_overlap(bounds[(size_t)v2 * g.N + i], x0, x1, y0, y1);
        if (nviews <= -4) keep |= rect_overlap(bounds[(size_t)v3 * g.N + i], x0, x1, y0, y1);
      }
    }
    const unsigned long long m = __ballot(keep);
    mine = (lane == r) ? m : mine;
    running += __popcll(m);
  }
  if (lane < kChunk / 64) masks[lane] = mine;
  if (lane == 0) l1_counts[s * g.NC + c] = (int32_t)running;
}

// The counting pass of level 1 for one view, in bands of at most kScatterMaxSuper super-tiles: by primitive
// instead of by (chunk, super-tile), and with the bounds computed on the way (every primitive is visited exactly
// once, so this is also the bounds kernel).  The walk above tests every primitive against every super-tile (N x S
// rectangle tests); here one workgroup per chunk lets each primitive find the few super-tiles it overlaps and set
// its bit in that super-tile's row of an LDS bitmap [S][kChunk bits].  The rows are the very ballots the walk
// produces: they are stored where the walk stores them, counted, and the walk's fill pass writes the lists from
// them (it writes consecutive list positions from consecutive lanes; a fill by primitive scatters 20-byte stores and
// measured slower).  Dynamic LDS: scatter_lds_bytes(S) -- the bitmap and the list of wide primitives.
constexpr int kScatterThreads = 1024;
constexpr int kScatterMaxSuper = 400;
constexpr int kWordsPerRow = kChunk / 64;
constexpr int kScatterWide = 2 * kChunk;     // entries of the list of wide (primitive, view) pairs
constexpr int kScatterMaxViews = 32;
__host__ __device__ constexpr size_t scatter_lds_bytes(int S) {
  return (size_t)S * (kWordsPerRow * sizeof(unsigned long long) + sizeof(unsigned)) + kScatterWide * sizeof(uint2);
}

// super-tile columns (rows) a [lo, hi] pixel interval overlaps under rect_overlap's strict inequalities: [a, b],
// empty when a > b.  n: super-tiles along the axis, nt: tiles along it.  Column k spans [x0(k), x1(k)) pixels and
// passes when lo < x1(k) and hi > x0(k); x0 and x1 grow with k, so a is the first k with lo < x1(k) and b the last
// with hi > x0(k).  Both are estimated from a division, moved by one where the comparison itself says so, and
// checked against their definition; the walk over all columns is the fallback that the check never asks for in
// practice but that makes the result exact whatever the rounding of the estimate.
__device__ __forceinline__ void super_range(float lo, float hi, int n, int nt, int ts, int& a, int& b) {
  a = 0;
  b = -1;
  if (lo != lo || hi != hi) return;      // behind the near plane: NaN bounds overlap nothing
  const float inv = 1.f / (float)(kSuper * ts);
  auto x0 = [&](int k) { return (float)(k * kSuper * ts); };
  auto x1 = [&](int k) { return (float)(min((k + 1) * kSuper, nt) * ts); };
  int ea = (int)fmaxf(fminf(floorf(lo * inv), (float)n), 0.f);
  if (ea > 0 && lo < x1(ea - 1)) --ea;
  else if (ea < n && !(lo < x1(ea))) ++ea;
  int eb = (int)fmaxf(fminf(floorf(hi * inv), (float)(n - 1)), -1.f);
  if (eb < n - 1 && hi > x0(eb + 1)) ++eb;
  else if (eb >= 0 && !(hi > x0(eb))) --eb;
  const bool a_ok = (ea == n || lo < x1(ea)) && (ea == 0 || !(lo < x1(ea - 1)));
  const bool b_ok = (eb == -1 || hi > x0(eb)) && (eb == n - 1 || !(hi > x0(eb + 1)));
  if (!(a_ok && b_ok)) {
    ea = n;
    eb = -1;
    for (int k = 0; k < n; ++k) {
      if ((lo < x1(k)) && (hi > x0(k))) {
        ea = min(ea, k);
        eb = k;
      }
    }
  }
  a = ea;
  b = eb;
}

// grid = (NC, bands): workgroup (c, band) handles chunk c and the super-tile rows [band * band_rows, + band_rows), so
// that the bitmap of any screen fits LDS (every band computes the chunk's bounds; band 0 stores them).
// MODE 1, 2: one view, bounds computed here (bin_bounds_kernel's modes).  MODE 0: several views (at most 32) with
// tile_view_ids; the bounds of all views come from bin_bounds_kernel, the workgroup first collects which views the
// tiles of each of its super-tiles use, and a primitive sets its bit in a super-tile when its rectangle under one of
// THOSE views overlaps it (the walk tests the same views, or all of them when a super-tile uses more than four: the
// lists are a superset either way, and level 2 applies each tile's own view).
template <int MODE>
__global__ __launch_bounds__(kScatterThreads) void bin_level1_scatter_kernel(
    const float* __restrict__ pos, const float* __restrict__ logs, const float* __restrict__ mats,
    const float* __restrict__ proj_dev, BinMats one, BinGeom g, float rm, float focal, int band_rows,
    const int32_t* __restrict__ tile_view_ids, float4* __restrict__ bounds, int32_t* __restrict__ l1_counts,
    int32_t* __restrict__ super_view, unsigned long long* __restrict__ l1_masks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
  const int row0 = blockIdx.y * band_rows, rows = min(band_rows, g.nsy - row0);
  const int S = g.nsx * rows;                          // super-tiles of this band; the first is row0 * nsx
  const int smax = g.nsx * band_rows;
  unsigned long long* __restrict__ bits = reinterpret_cast<unsigned long long*>(s_raw);      // [S][kWordsPerRow]
  // wide primitives: (p | view << 16, xa xb ya yb one byte each, ya and yb counted from row0)
  uint2* __restrict__ wide = reinterpret_cast<uint2*>(bits + (size_t)smax * kWordsPerRow);
  unsigned* __restrict__ views = reinterpret_cast<unsigned*>(wide + kScatterWide);            // [S] (MODE 0)
  __shared__ int s_nwide;
  const int c = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  for (int w = t; w < S * kWordsPerRow; w += kScatterThreads) bits[w] = 0ull;
  if (MODE == 0)
    for (int k = t; k < S; k += kScatterThreads) views[k] = 0u;
  if (t == 0) s_nwide = 0;
  __syncthreads();
  if (MODE == 0) {
    // one item = one row of 8 tiles of a super-tile
    for (int item = t; item < S * kSuper; item += kScatterThreads) {
      const int sl = item / kSuper, ty = (row0 + sl / g.nsx) * kSuper + item % kSuper, tx0 = (sl % g.nsx) * kSuper;
      unsigned m = 0u;
      if (ty < g.nty) {
#pragma unroll
        for (int j = 0; j < kSuper; ++j) {
          const int v = (tx0 + j < g.ntx) ? tile_view_ids[ty * g.ntx + tx0 + j] : -1;
          m |= ((unsigned)v < (unsigned)g.K) ? (1u << v) : 0u;
        }
      }
      if (m) atomicOr(&views[sl], m);
    }
    __syncthreads();
  }
  // A primitive that overlaps more than kNarrow super-tiles is not walked by its own thread (the workgroup would wait
  // for the few threads that hold such primitives): it goes on a list, and a whole wavefront walks its super-tiles.
  constexpr int kNarrow = 4;
  constexpr int kPer = kChunk / kScatterThreads;     // primitives per thread
  auto mark = [&](int cell, int p, int view) {
    if (MODE != 0 || ((views[cell] >> view) & 1u))
      atomicOr(&bits[(size_t)cell * kWordsPerRow + (p >> 6)], 1ull << (p & 63));
  };
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int p = t + u * kScatterThreads, i = c * kChunk + p;
    if (i < g.N) {
      for (int view = 0; view < (MODE == 0 ? g.K : 1); ++view) {
        float4 bb;
        if (MODE == 0) {
          bb = bounds[(size_t)view * g.N + i];
        } else {
          bb = primitive_bounds<MODE>(pos, logs, mats, proj_dev, one, g, rm, focal, i, 0);
          if (blockIdx.y == 0) bounds[i] = bb;
        }
        int xa, xb, ya, yb;
        super_range(bb.x, bb.y, g.nsx, g.ntx, g.ts, xa, xb);
        super_range(bb.z, bb.w, g.nsy, g.nty, g.ts, ya, yb);
        ya = max(ya, row0) - row0;           // rows of this band only, counted from its first row
        yb = min(yb, row0 + rows - 1) - row0;
        if (xa > xb) yb = ya - 1;            // (no column: no row either)
        if ((xb - xa + 1) * (yb - ya + 1) > kNarrow) {
          const int slot = atomicAdd(&s_nwide, 1);
          if (slot < kScatterWide) {         // (a full list: the thread walks the primitive after all)
            wide[slot] = make_uint2((unsigned)p | ((unsigned)view << 16), (unsigned)xa | ((unsigned)xb << 8) |
                                                                              ((unsigned)ya << 16) | ((unsigned)yb << 24));
            yb = ya - 1;
          }
        }
        for (int sy = ya; sy <= yb; ++sy)
          for (int sx = xa; sx <= xb; ++sx) mark(sy * g.nsx + sx, p, view);
      }
    }
  }
  __syncthreads();
  const int nwide = min(s_nwide, kScatterWide);
  for (int e = wave; e < nwide; e += kScatterThreads / 64) {
    const uint2 we = wide[e];
    const int p = (int)(we.x & 0xffffu), view = (int)(we.x >> 16);
    const int wxa = we.y & 255, wxb = (we.y >> 8) & 255, wya = (we.y >> 16) & 255, wyb = we.y >> 24;
    const int nx = wxb - wxa + 1, cells = nx * (wyb - wya + 1);
    for (int k = lane; k < cells; k += 64) mark((wya + k / nx) * g.nsx + wxa + k % nx, p, view);
  }
  __syncthreads();
  // 32 lanes per row: lane w of the group holds word w of the row
  static_assert(kWordsPerRow == 32, "a row is handled by half a wavefront");
  const int w = t & 31, first = row0 * g.nsx;
  for (int row = t >> 5; row < S; row += kScatterThreads / 32) {
    const unsigned long long word = bits[(size_t)row * kWordsPerRow + w];
    l1_masks[((size_t)(first + row) * g.NC + c) * kWordsPerRow + w] = word;
    int n = __popcll(word);
#pragma unroll
    for (int d = 16; d >= 1; d >>= 1) n += __shfl_xor(n, d);
    if (w == 0) l1_counts[(first + row) * g.NC + c] = n;
  }
  if (c == 0) {
    for (int k = t; k < S; k += kScatterThreads) {
      const unsigned m = MODE == 0 ? views[k] : 1u;
      super_view[first + k] = (__popc(m) == 1) ? (int)__builtin_ctz(m) : -1;
    }
  }
}

// level 1, fill pass for one (chunk, super-tile) pair by one wavefront; `running` is where the pair's survivors
// start in the level-1 list.  The counting pass left one ballot per 64 primitives: no bounds are read again except
// the survivors'.  Lane r fetches ballot r (one coalesced load), the ballots' bit counts are scanned, and then lane
// k writes the k-th survivor: it finds the ballot that holds it (a search over the scanned counts) and the bit
// inside.  All survivors' bounds are gathered at once -- one memory latency per 64 survivors; walking the ballots
// one after the other instead costs one per ballot that is not empty.
__device__ __forceinline__ unsigned long long level1_ballots(const BinGeom& g, int c, int s,
                                                             const unsigned long long* __restrict__ l1_masks) {
  const int lane = threadIdx.x & 63;
  return lane < kChunk / 64 ? l1_masks[((size_t)s * g.NC + c) * (kChunk / 64) + lane] : 0ull;
}
__device__ __forceinline__ void level1_fill_pair(int c, unsigned long long mine, long long running, bool single,
                                                 const float4* __restrict__ sb, int32_t* __restrict__ l1_list,
                                                 float4* __restrict__ l1_bounds, long long l1_capacity) {
  const int lane = threadIdx.x & 63;
  const int first = c * kChunk;
  const int own = __popcll(mine);
  int incl = own;
#pragma unroll
  for (int d = 1; d < kChunk / 64; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  const int before = incl - own;                     // survivors in the ballots ahead of this lane's
  const int total = __shfl(incl, kChunk / 64 - 1);
  static_assert(kChunk / 64 == 32, "the search below halves 32 ballots");
  for (int k0 = 0; k0 < total; k0 += 64) {
    const int k = k0 + lane;
    int r = 0;                                       // the last ballot whose `before` is <= k holds survivor k
#pragma unroll
    for (int step = 16; step >= 1; step >>= 1) {
      const int ahead = __shfl(before, r + step);
      if (ahead <= k) r += step;
    }
    const int nth = k - __shfl(before, r);
    const unsigned long long m = ((unsigned long long)(unsigned)__shfl((int)(mine >> 32), r) << 32) |
                                 (unsigned)__shfl((int)mine, r);
    if (k < total) {
      const int i = first + r * 64 + nth_set_bit(m, nth);
      const long long dst = running + k;
      if (dst < l1_capacity) {
        l1_list[dst] = i;
        if (single) l1_bounds[dst] = sb[i];
      }
    }
  }
}

__device__ __forceinline__ long long wave_sum(long long x) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d);
  return x;
}

// level 1, fill pass.  grid = S workgroups of 1024 threads: workgroup s writes super-tile s's list, chunk after chunk
// (ascending primitive ids), a wavefront per (chunk, super-tile) pair.  Lists follow each other in super-tile order, so
// the list starts where the counts of all super-tiles before it add up to: the workgroup adds them up itself (a
// coalesced read of s * NC counts, all requested before the first is used; a scan kernel between the passes cost a
// launch in a chain of dependent launches, ~10 us, for the same sums; a row split over several workgroups repeats
// this read and measured slower), then scans its own row of counts.  l1_super[s] receives the start of list s and
// l1_super[S] the end of the last one (both clamped to the capacity, like every store to the list), totals[0] the
// unclamped number of entries.
__global__ __launch_bounds__(kWideThreads) void bin_level1_fill_kernel(
    const float4* __restrict__ bounds, BinGeom g, const int32_t* __restrict__ l1_counts,
    int32_t* __restrict__ l1_list, float4* __restrict__ l1_bounds, long long l1_capacity,
    const unsigned long long* __restrict__ l1_masks, const int32_t* __restrict__ super_view,
    int32_t* __restrict__ l1_super, long long* __restrict__ totals, long long* __restrict__ clear_word) {
  __shared__ long long s_part[kWideThreads / 64];
  __shared__ long long s_start[kWideThreads];
  const int s = blockIdx.x, S = g.nsx * g.nsy;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const long long n_before = (long long)s * g.NC;
  // the ballots of the wavefront's first pairs do not depend on where the list starts: requested ahead of the sums
  constexpr int kAhead = 8;
  unsigned long long ahead[kAhead];
#pragma unroll
  for (int j = 0; j < kAhead; ++j) {
    const int c = wave + j * (kWideThreads / 64);
    ahead[j] = (c < g.NC) ? level1_ballots(g, c, s, l1_masks) : 0ull;      // (uniform per wavefront)
  }
  // eight 16-byte loads in flight per thread and step.  (The array is 256-byte aligned and its size a multiple of
  // that: the four ints at a multiple of 4 below n_before all lie inside it; those at or beyond n_before are dropped.)
  long long acc = 0;
  for (long long i0 = (long long)t * 4; i0 < n_before; i0 += 8 * 4 * kWideThreads) {
    int4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const long long i = i0 + (long long)u * 4 * kWideThreads;
      // (a load beyond the end reads the array's first ints instead and is dropped below: a load under a condition
      // would wait for the one before it)
      v[u] = *reinterpret_cast<const int4*>(l1_counts + ((i < n_before) ? i : 0));
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const long long i = i0 + (long long)u * 4 * kWideThreads;
      acc += (i < n_before) ? v[u].x : 0;
      acc += (i + 1 < n_before) ? v[u].y : 0;
      acc += (i + 2 < n_before) ? v[u].z : 0;
      acc += (i + 3 < n_before) ? v[u].w : 0;
    }
  }
  acc = wave_sum(acc);
  if (lane == 0) s_part[wave] = acc;
  __syncthreads();
  long long base = 0;
#pragma unroll
  for (int w = 0; w < kWideThreads / 64; ++w) base += s_part[w];
  const int view = super_view[s];
  const bool single = view >= 0;
  const float4* __restrict__ sb = bounds + (size_t)(single ? view : 0) * g.N;
  const int32_t* __restrict__ row = l1_counts + (size_t)s * g.NC;
  long long carry = base;
  for (int c0 = 0; c0 < g.NC; c0 += kWideThreads) {
    const int own = (c0 + t < g.NC) ? row[c0 + t] : 0;
    long long incl = own;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const long long up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    __syncthreads();                                  // (s_part and s_start are free again)
    if (lane == 63) s_part[wave] = incl;
    __syncthreads();
    long long before = carry, pass_total = 0;
#pragma unroll
    for (int w = 0; w < kWideThreads / 64; ++w) {
      const long long n = s_part[w];
      before += (w < wave) ? n : 0;
      pass_total += n;
    }
    s_start[t] = before + incl - own;
    __syncthreads();
    const int here = min(g.NC - c0, kWideThreads);
    if (c0 == 0) {
#pragma unroll
      for (int j = 0; j < kAhead; ++j) {
        const int k = wave + j * (kWideThreads / 64);
        if (k < here) level1_fill_pair(k, ahead[j], s_start[k], single, sb, l1_list, l1_bounds, l1_capacity);
      }
    }
    for (int k = wave + (c0 == 0 ? kAhead * (kWideThreads / 64) : 0); k < here; k += kWideThreads / 64)
      level1_fill_pair(c0 + k, level1_ballots(g, c0 + k, s, l1_masks), s_start[k], single, sb, l1_list, l1_bounds,
                       l1_capacity);
    carry += pass_total;
  }
  if (t == 0) {
    l1_super[s] = (int32_t)min(base, l1_capacity);
    if (s == S - 1) {
      l1_super[S] = (int32_t)min(carry, l1_capacity);
      totals[0] = carry;
      if (clear_word) *clear_word = 0;      // (the segment form of level 2, the next launch, takes maxima into it)
    }
  }
}

// In-place exclusive scan of data[0..n) by one workgroup; data[n] and *total receive the sum, *largest
// (if not null) the largest element.  data must be 16-byte aligned.  A pass covers 8 slabs of 4096
// elements: thread t owns elements 4t..4t+3 of every slab, so all loads and stores are coalesced 16-byte
// accesses and the 8 loads of a pass are independent (one memory latency per pass, and one pass covers
// 32768 elements).  Thread sums are scanned with wavefront shuffles, wavefront totals through LDS.
// (Only the two-call binning, whose caller sizes the candidate buffer from the total, scans with a kernel of its
// own; the asynchronous entry points place their lists inside the fill passes.)
constexpr int kScanSlabs = 8;
__global__ __launch_bounds__(1024) void exclusive_scan_kernel(int32_t* __restrict__ data, int n,
                                                              long long* __restrict__ total,
                                                              long long* __restrict__ largest) {
  __shared__ long long s_wave[kScanSlabs][16];
  __shared__ int s_wmax[16];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  long long carry = 0;
  int mx = 0;
  for (int pass0 = 0; pass0 < n; pass0 += kScanSlabs * 4096) {
    int4 v[kScanSlabs];
#pragma unroll
    for (int u = 0; u < kScanSlabs; ++u) {
      const int idx = pass0 + u * 4096 + t * 4;
      if (idx + 3 < n) {
        v[u] = *reinterpret_cast<const int4*>(data + idx);
      } else {
        v[u].x = (idx < n) ? data[idx] : 0;
        v[u].y = (idx + 1 < n) ? data[idx + 1] : 0;
        v[u].z = (idx + 2 < n) ? data[idx + 2] : 0;
        v[u].w = 0;
      }
    }
    long long incl[kScanSlabs];
#pragma unroll
    for (int u = 0; u < kScanSlabs; ++u) {
      incl[u] = 0;
      if (pass0 + u * 4096 >= n) {            // slab beyond the data (workgroup-uniform): nothing to scan
        if (lane == 63) s_wave[u][wave] = 0;
        continue;
      }
      mx = max(max(mx, max(v[u].x, v[u].y)), max(v[u].z, v[u].w));
      long long x = (long long)v[u].x + v[u].y + v[u].z + v[u].w;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const long long up = __shfl_up(x, d);
        if (lane >= d) x += up;
      }
      incl[u] = x;
      if (lane == 63) s_wave[u][wave] = x;
    }
    __syncthreads();
    long long base = carry;
#pragma unroll
    for (int u = 0; u < kScanSlabs; ++u) {
      if (pass0 + u * 4096 >= n) continue;
      long long before = 0, slab = 0;
#pragma unroll
      for (int w = 0; w < 16; ++w) {
        const long long c = s_wave[u][w];
        before += (w < wave) ? c : 0;
        slab += c;
      }
      const long long own = (long long)v[u].x + v[u].y + v[u].z + v[u].w;
      const long long e0 = base + before + incl[u] - own;
      const int idx = pass0 + u * 4096 + t * 4;
      const int4 o = make_int4((int)e0, (int)(e0 + v[u].x), (int)(e0 + v[u].x + v[u].y),
                               (int)(e0 + v[u].x + v[u].y + v[u].z));
      if (idx + 3 < n) {
        *reinterpret_cast<int4*>(data + idx) = o;
      } else {
        if (idx < n) data[idx] = o.x;
        if (idx + 1 < n) data[idx + 1] = o.y;
        if (idx + 2 < n) data[idx + 2] = o.z;
      }
      base += slab;
    }
    carry = base;
    __syncthreads();
  }
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) mx = max(mx, __shfl_xor(mx, d));
  if (lane == 0) s_wmax[wave] = mx;
  __syncthreads();
  if (t == 0) {
    int all_max = 0;
    for (int w = 0; w < 16; ++w) all_max = max(all_max, s_wmax[w]);
    data[n] = (int32_t)carry;
    *total = carry;
    if (largest) *largest = all_max;
  }
}

// level 2.  One wavefront per tile.  Ballot b of a tile lives at [tile within its super-tile][lo / 64 + s + b]:
// super-tile lists are consecutive in the level-1 array, so adding s keeps the slots of neighbouring lists apart.
struct L2Tile {
  int lo, hi, nb, s, view;
  float x0, x1, y0, y1;
  unsigned long long* masks;
};
__device__ __forceinline__ L2Tile level2_tile(const BinGeom& g, int tile, const int32_t* __restrict__ tile_view_ids,
                                              const int32_t* __restrict__ l1_super, long long l1_capacity,
                                              unsigned long long* __restrict__ l2_masks, long long l2_mask_stride) {
  L2Tile t;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  t.s = (ty / kSuper) * g.nsx + (tx / kSuper);
  t.view = tile_view_ids ? tile_view_ids[tile] : 0;
  t.x0 = (float)(tx * g.ts);
  t.x1 = (float)((tx + 1) * g.ts);
  t.y0 = (float)(ty * g.ts);
  t.y1 = (float)((ty + 1) * g.ts);
  // clamped so that an overflowed level-1 list (reported to the host) is never read past its end
  t.lo = (int)min((long long)l1_super[t.s], l1_capacity);
  t.hi = (int)min((long long)l1_super[t.s + 1], l1_capacity);
  t.hi = max(t.hi, t.lo);
  t.nb = (t.hi - t.lo + 63) >> 6;
  t.masks = l2_masks + (size_t)((ty % kSuper) * kSuper + (tx % kSuper)) * l2_mask_stride + (t.lo >> 6) + t.s;
  return t;
}

// counting pass of one tile: tests its super-tile's list, keeps the ballots, returns the number of survivors
__device__ __forceinline__ int level2_count_tile(const L2Tile& t, const BinGeom& g, const float4* __restrict__ bounds,
                                                 const int32_t* __restrict__ l1_list,
                                                 const float4* __restrict__ l1_bounds,
                                                 const int32_t* __restrict__ super_view) {
  const int lane = threadIdx.x & 63;
  const int lo = t.lo, hi = t.hi, nb = t.nb;
  const float x0 = t.x0, x1 = t.x1, y0 = t.y0, y1 = t.y1;
  unsigned long long* __restrict__ masks = t.masks;
  int running = 0;
  unsigned long long mine = 0ull;
  if (super_view[t.s] == t.view) {
    // one view for the super-tile: its bounds sit next to the ids; four independent 16-byte loads in flight per step
    const float nanv = __builtin_nanf("");
    for (int b = 0; b < nb; b += 4) {
      float4 bb[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = lo + ((b + u) << 6) + lane;
        bb[u] = (j < hi) ? l1_bounds[j] : make_float4(nanv, nanv, nanv, nanv);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (b + u < nb) {
          const unsigned long long m = __ballot(rect_overlap(bb[u], x0, x1, y0, y1));
          mine = (lane == ((b + u) & 63)) ? m : mine;
          if (((b + u) & 63) == 63) masks[b + u - 63 + lane] = mine;
          running += __popcll(m);
        }
      }
    }
  } else {
    const float4* __restrict__ vb = bounds + (size_t)t.view * g.N;
    for (int base = lo, b = 0; base < hi; base += 64, ++b) {
      const int j = base + lane;
      bool keep = false;
      if (j < hi) keep = rect_overlap(vb[l1_list[j]], x0, x1, y0, y1);
      const unsigned long long m = __ballot(keep);
      mine = (lane == (b & 63)) ? m : mine;
      if ((b & 63) == 63) masks[b - 63 + lane] = mine;       // 64 ballots at a time, one coalesced store
      running += __popcll(m);
    }
  }
  if ((nb & 63) != 0 && lane < (nb & 63)) masks[(nb & ~63) + lane] = mine;
  return running;
}

// fill pass of one tile: its survivors' ids, from the ballots, to cand[running...]
// (first: the tile's first 64 ballots, lane b holding ballot b -- the caller requests them ahead of time)
__device__ __forceinline__ unsigned long long level2_first_ballots(const L2Tile& t) {
  const int lane = threadIdx.x & 63;
  return (lane < t.nb) ? t.masks[lane] : 0ull;
}
__device__ __forceinline__ void level2_fill_tile(const L2Tile& t, unsigned long long first,
                                                 const int32_t* __restrict__ l1_list, int32_t* __restrict__ cand,
                                                 int running) {
  const int lane = threadIdx.x & 63;
  const int lo = t.lo, nb = t.nb;
  const unsigned long long* __restrict__ masks = t.masks;
  for (int b0 = 0; b0 < nb; b0 += 64) {         // 64 ballots per coalesced load, lane b holds ballot b0 + b
    const unsigned long long mine = (b0 == 0) ? first : (b0 + lane < nb) ? masks[b0 + lane] : 0ull;
    const int nhere = min(64, nb - b0);
    for (int b = 0; b < nhere; b += 8) {        // eight ballots at a time: their id loads are in flight together
      unsigned long long m[8];
      int id[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) m[u] = (b + u < nhere) ? lane_value(mine, (b + u) & 63) : 0ull;
#pragma unroll
      for (int u = 0; u < 8; ++u) id[u] = ((m[u] >> lane) & 1ull) ? l1_list[lo + ((b0 + b + u) << 6) + lane] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if ((m[u] >> lane) & 1ull) cand[running + lanes_below(m[u])] = id[u];
        running += __popcll(m[u]);
      }
    }
  }
}

// level 2, counting pass: 16 tiles per workgroup.  tile_counts[tile] = survivors, groups[workgroup] = their sum and
// the longest of the 16 lists.
__global__ __launch_bounds__(kWideThreads) void bin_level2_count_kernel(
    const float4* __restrict__ bounds, BinGeom g, const int32_t* __restrict__ tile_view_ids,
    const int32_t* __restrict__ l1_super, const int32_t* __restrict__ l1_list, const float4* __restrict__ l1_bounds,
    long long l1_capacity, int32_t* __restrict__ tile_counts, unsigned long long* __restrict__ l2_masks,
    long long l2_mask_stride, const int32_t* __restrict__ super_view, L2Group* __restrict__ groups) {
  __shared__ int s_cnt[kL2Group];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tile = blockIdx.x * kL2Group + wave;
  int count = 0;
  if (tile < g.ntx * g.nty) {
    const L2Tile t = level2_tile(g, tile, tile_view_ids, l1_super, l1_capacity, l2_masks, l2_mask_stride);
    count = level2_count_tile(t, g, bounds, l1_list, l1_bounds, super_view);
    if (lane == 0) tile_counts[tile] = count;
  }
  if (lane == 0) s_cnt[wave] = count;
  __syncthreads();
  if (threadIdx.x == 0) {
    L2Group grp;
    grp.sum = 0;
    grp.longest = 0;
    grp.pad = 0;
#pragma unroll
    for (int w = 0; w < kL2Group; ++w) {
      grp.sum += s_cnt[w];
      grp.longest = max(grp.longest, s_cnt[w]);
    }
    groups[blockIdx.x] = grp;
  }
}

// level 2, fill pass: the same 16 tiles per workgroup.
// OWN_PREFIX = false: tile_offsets holds the exclusive offsets (the caller scanned the counts).
// OWN_PREFIX = true: tile_offsets holds the counts, and the workgroup places its tiles itself -- it adds up the
// groups before its own (a few KB that are L2 hits, instead of a scan kernel between the passes), every workgroup
// also forms the total and applies the guard of the asynchronous entry points: if the level-1 lists overflowed their
// scratch (totals[0] > l1_capacity) or the total does not fit the caller's candidate buffer, every offset is written
// as 0, nothing is filled and the guard word totals[3] is raised, so that the sort and render kernels queued behind
// find nothing to read or write; counts_out receives (pairs, longest list, level-1 entries, guard).  A workgroup
// reads only its own tiles' counts before it overwrites them with offsets.
struct FillGuard {
  long long* totals;
  long long* counts_out;
  long long l1_capacity, cand_capacity;
};
template <bool OWN_PREFIX>
__global__ __launch_bounds__(kWideThreads) void bin_level2_fill_kernel(
    BinGeom g, const int32_t* __restrict__ tile_view_ids, const int32_t* __restrict__ l1_super,
    const int32_t* __restrict__ l1_list, long long l1_capacity, int32_t* __restrict__ tile_offsets,
    int32_t* __restrict__ cand, unsigned long long* __restrict__ l2_masks, long long l2_mask_stride,
    const L2Group* __restrict__ groups, int num_groups, FillGuard guard) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int T = g.ntx * g.nty;
  const int tile = blockIdx.x * kL2Group + wave;
  int running = 0;
  // (what does not depend on the tile's place is requested first: the list bounds, the first ballots)
  L2Tile tl = {};
  unsigned long long first = 0ull;
  if (tile < T) {
    tl = level2_tile(g, tile, tile_view_ids, l1_super, l1_capacity, l2_masks, l2_mask_stride);
    first = level2_first_ballots(tl);
  }
  if constexpr (OWN_PREFIX) {
    __shared__ long long s_before[kL2Group], s_total[kL2Group];
    __shared__ int s_longest[kL2Group], s_cnt[kL2Group];
    const long long l1_entries = guard.totals[0];      // (requested up front)
    long long before = 0, total = 0;
    int longest = 0;
    for (int k0 = threadIdx.x; k0 < num_groups; k0 += 4 * kWideThreads) {      // four loads in flight
      L2Group v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + u * kWideThreads;
        v[u] = groups[(k < num_groups) ? k : 0];      // (unconditional, so that the four do not wait for each other)
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + u * kWideThreads;
        total += (k < num_groups) ? v[u].sum : 0;
        before += (k < (int)blockIdx.x) ? v[u].sum : 0;
        longest = max(longest, (k < num_groups) ? v[u].longest : 0);
      }
    }
    const int own = (tile < T) ? tile_offsets[tile] : 0;
    before = wave_sum(before);
    total = wave_sum(total);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) longest = max(longest, __shfl_xor(longest, d));
    if (lane == 0) {
      s_before[wave] = before;
      s_total[wave] = total;
      s_longest[wave] = longest;
      s_cnt[wave] = own;
    }
    __syncthreads();
    before = 0;
    total = 0;
    longest = 0;
#pragma unroll
    for (int w = 0; w < kL2Group; ++w) {
      before += s_before[w] + ((w < wave) ? s_cnt[w] : 0);
      total += s_total[w];
      longest = max(longest, s_longest[w]);
    }
    const bool bad = l1_entries > guard.l1_capacity || total > guard.cand_capacity;
    if (lane == 0) {
      if (tile < T) tile_offsets[tile] = bad ? 0 : (int32_t)before;
      if (tile == T - 1) tile_offsets[T] = bad ? 0 : (int32_t)total;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      guard.totals[1] = total;
      guard.totals[2] = longest;
      guard.totals[3] = bad ? 1 : 0;
      guard.counts_out[0] = total;
      guard.counts_out[1] = longest;
      guard.counts_out[2] = l1_entries;
      guard.counts_out[3] = bad ? 1 : 0;
    }
    if (bad || tile >= T) return;
    running = (int)before;
  } else {
    if (tile >= T) return;
    running = tile_offsets[tile];
  }
  level2_fill_tile(tl, first, l1_list, cand, running);
}

// level 2 in one pass, into segments: tile t owns cand[t * stride .. (t + 1) * stride) and its list is the first
// ends[t] - t * stride entries of it.  No counting pass and no placing: a wavefront tests its tile's super-tile list 64
// entries at a time and appends the survivors where its own count stands.  What the lists of a frame lose in
// compactness they never needed: the sort and the render read a tile's list from its start to its end.  `stride` is
// the tile capacity of the render path; a tile with more survivors keeps the first `stride` and reports its length
// into *longest (a maximum; cleared by the level-1 fill launch), which the caller turns into the capacity error.
// tile_offsets[t] = t * stride (T + 1 of them).  If the level-1 lists overflowed their scratch every list is left
// empty and the guard word is raised, as in bin_level2_fill_kernel<true>; counts_out = (0, longest if over the
// capacity, level-1 entries, guard).
__device__ __forceinline__ int level2_segment_tile(const L2Tile& t, const BinGeom& g, const float4* __restrict__ bounds,
                                                   const int32_t* __restrict__ l1_list,
                                                   const float4* __restrict__ l1_bounds,
                                                   const int32_t* __restrict__ super_view, int32_t* __restrict__ seg,
                                                   int stride) {
  const int lane = threadIdx.x & 63;
  const int lo = t.lo, hi = t.hi, nb = t.nb;
  const float x0 = t.x0, x1 = t.x1, y0 = t.y0, y1 = t.y1;
  int running = 0;
  if (super_view[t.s] == t.view) {
    const float nanv = __builtin_nanf("");
    for (int b = 0; b < nb; b += 4) {
      float4 bb[4];
      int id[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = lo + ((b + u) << 6) + lane;
        bb[u] = (j < hi) ? l1_bounds[j] : make_float4(nanv, nanv, nanv, nanv);
        id[u] = (j < hi) ? l1_list[j] : 0;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (b + u < nb) {
          const bool keep = rect_overlap(bb[u], x0, x1, y0, y1);
          const unsigned long long m = __ballot(keep);
          const int at = running + lanes_below(m);
          if (keep && at < stride) seg[at] = id[u];
          running += __popcll(m);
        }
      }
    }
  } else {
    const float4* __restrict__ vb = bounds + (size_t)t.view * g.N;
    for (int base = lo; base < hi; base += 64) {
      const int j = base + lane;
      bool keep = false;
      int id = 0;
      if (j < hi) {
        id = l1_list[j];
        keep = rect_overlap(vb[id], x0, x1, y0, y1);
      }
      const unsigned long long m = __ballot(keep);
      const int at = running + lanes_below(m);
      if (keep && at < stride) seg[at] = id;
      running += __popcll(m);
    }
  }
  return running;
}

__global__ __launch_bounds__(kWideThreads) void bin_level2_segments_kernel(
    const float4* __restrict__ bounds, BinGeom g, const int32_t* __restrict__ tile_view_ids,
    const int32_t* __restrict__ l1_super, const int32_t* __restrict__ l1_list, const float4* __restrict__ l1_bounds,
    long long l1_capacity, unsigned long long* __restrict__ l2_masks, long long l2_mask_stride,
    const int32_t* __restrict__ super_view, const long long* __restrict__ totals, int stride,
    int32_t* __restrict__ tile_offsets, int32_t* __restrict__ tile_ends, int32_t* __restrict__ cand,
    long long* __restrict__ counts_out) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int T = g.ntx * g.nty;
  const int tile = blockIdx.x * kL2Group + wave;
  const long long l1_entries = totals[0];
  const bool bad = l1_entries > l1_capacity;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    counts_out[0] = 0;
    counts_out[2] = l1_entries;
    counts_out[3] = bad ? 1 : 0;
  }
  if (tile >= T) return;
  const int start = tile * stride;
  if (lane == 0) {
    tile_offsets[tile] = start;
    if (tile == T - 1) tile_offsets[T] = T * stride;
  }
  int count = 0;
  if (!bad) {
    const L2Tile t = level2_tile(g, tile, tile_view_ids, l1_super, l1_capacity, l2_masks, l2_mask_stride);
    count = level2_segment_tile(t, g, bounds, l1_list, l1_bounds, super_view, cand + start, stride);
  }
  if (lane == 0) {
    tile_ends[tile] = start + min(count, stride);
    if (count > stride) atomicMax(reinterpret_cast<unsigned long long*>(counts_out + 1), (unsigned long long)count);
  }
}

inline BinGeom make_geom(int N, int K, int W, int H, int ts) {
  BinGeom g;
  g.W = W; g.H = H; g.ts = ts;
  g.ntx = ceil_div(W, ts); g.nty = ceil_div(H, ts);
  g.nsx = ceil_div(g.ntx, kSuper); g.nsy = ceil_div(g.nty, kSuper);
  g.N = N; g.K = K; g.NC = ceil_div(N > 0 ? N : 1, kChunk);
  return g;
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_bin_scratch_bytes(int num_primitives, int num_views, int width, int height, int tile) {
  if (num_primitives < 0 || num_views <= 0 || checked_num_tiles(width, height, tile, tile) <= 0) return 0;
  const BinGeom g = make_geom(num_primitives, num_views, width, height, tile);
  const size_t S = (size_t)g.nsx * g.nsy;
  size_t bytes = align256((size_t)(num_views + 1) * 16 * sizeof(float)) +
                 align256((size_t)num_views * num_primitives * sizeof(float4)) +
                 align256((S * g.NC + 1) * sizeof(int32_t)) + 256;
  bytes += align256(S * g.NC * (kChunk / 64) * sizeof(unsigned long long)) + align256(S * sizeof(int32_t));
  bytes += align256((S + 1) * sizeof(int32_t)) + align256((S * (64 / kL2Group) + 1) * sizeof(L2Group));
  bytes += 1024 + align256((S + 1) * 64 * sizeof(unsigned long long));
  // room for every primitive to touch 8 super-tiles per view, plus slack for tiny scenes; per entry the id,
  // the bounds and the 64 survivor bits of the super-tile's tiles
  const size_t entry = sizeof(int32_t) + sizeof(float4) + 8;
  bytes += align256(((size_t)8 * num_views * num_primitives + 65536) * entry) + 1024;
  return bytes;
}

namespace {
// MLPSP_BIN_LEVEL1_WALK=1 keeps the counting pass of level 1 on the (chunk, super-tile) walk where the by-primitive
// kernel would apply (for comparing the two; read once)
bool level1_walk_forced() {
  static const bool forced = [] {
    const char* v = getenv("MLPSP_BIN_LEVEL1_WALK");
    return v && v[0] == '1';
  }();
  return forced;
}

// the by-primitive counting kernel uses more dynamic LDS than a kernel may without saying so: said once per device
int allow_scatter_lds() {
  constexpr int kMaxDevices = 64;
  static bool done[kMaxDevices];
  int dev = -1;
  MLPSP_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return MLPSP_E_ARGUMENT;
  if (!__atomic_load_n(&done[dev], __ATOMIC_ACQUIRE)) {
    const int bytes = (int)scatter_lds_bytes(kScatterMaxSuper);
    MLPSP_HIP_TRY(hipFuncSetAttribute((const void*)bin_level1_scatter_kernel<0>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    MLPSP_HIP_TRY(hipFuncSetAttribute((const void*)bin_level1_scatter_kernel<1>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    MLPSP_HIP_TRY(hipFuncSetAttribute((const void*)bin_level1_scatter_kernel<2>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    __atomic_store_n(&done[dev], true, __ATOMIC_RELEASE);
  }
  return MLPSP_OK;
}

inline int level2_groups(int64_t T) { return (int)((T + kL2Group - 1) / kL2Group); }

// what the bounds of a frame are computed from (bin_bounds_kernel's arguments)
struct BoundsSource {
  const float* positions;
  const float* log_scales;
  int mode;                 // bin_bounds_kernel's MODE
  const float* mats;        // mode 0: K views then the projection; mode 2: the view matrix
  const float* proj_dev;    // mode 2
  BinMats one;              // mode 1
  float rm, focal;
};

// bounds -> level 1 (count, fill) -> level 2 count [-> scan of the tile counts when the caller fills separately]
// count_tiles = false stops after level 1 (the segment form of level 2 follows, which counts and fills in one pass
// and takes its maxima into *clear_word, cleared here).
int enqueue_bin_levels(const BoundsSource& src, const BinGeom& g, const BinScratch& b, int64_t T,
                       const int32_t* tile_view_ids_dev, int32_t* tile_offsets_dev, hipStream_t s, bool scan_tiles,
                       bool count_tiles = true, long long* clear_word = nullptr) {
  const int S = g.nsx * g.nsy;
  // level-1 counts by primitive (super-tile rows in bands that fit LDS): with one view the same launch computes the
  // bounds, with several (and tile_view_ids) it reads them
  const bool one_view = g.K == 1 && src.mode != 0;
  const bool many_views = src.mode == 0 && g.K > 1 && g.K <= kScatterMaxViews && tile_view_ids_dev != nullptr;
  const bool scatter = (one_view || many_views) && g.nsx <= kScatterMaxSuper && g.nsx < 256 && !level1_walk_forced();
  if (!scatter || many_views) {
    const dim3 grid(ceil_div(g.N, kBinThreads), src.mode == 0 ? g.K : 1), block(kBinThreads);
    if (src.mode == 0)
      hipLaunchKernelGGL(bin_bounds_kernel<0>, grid, block, 0, s, src.positions, src.log_scales, src.mats, src.proj_dev,
                         src.one, g, src.rm, src.focal, b.bounds);
    else if (src.mode == 1)
      hipLaunchKernelGGL(bin_bounds_kernel<1>, grid, block, 0, s, src.positions, src.log_scales, src.mats, src.proj_dev,
                         src.one, g, src.rm, src.focal, b.bounds);
    else
      hipLaunchKernelGGL(bin_bounds_kernel<2>, grid, block, 0, s, src.positions, src.log_scales, src.mats, src.proj_dev,
                         src.one, g, src.rm, src.focal, b.bounds);
    MLPSP_LAUNCH_CHECK();
  }
  if (scatter) {
    const int rc = allow_scatter_lds();
    if (rc != MLPSP_OK) return rc;
    const int band_rows = min(min(g.nsy, kScatterMaxSuper / g.nsx), 255);
    const size_t lds = scatter_lds_bytes(g.nsx * band_rows);
    const dim3 grid(g.NC, ceil_div(g.nsy, band_rows));
#define MLPSP_SCATTER(M)                                                                                             \
  hipLaunchKernelGGL(bin_level1_scatter_kernel<M>, grid, dim3(kScatterThreads), lds, s, src.positions, src.log_scales, \
                     src.mats, src.proj_dev, src.one, g, src.rm, src.focal, band_rows, tile_view_ids_dev, b.bounds,    \
                     b.l1_counts, b.super_view, b.l1_masks)
    if (src.mode == 0) MLPSP_SCATTER(0);
    else if (src.mode == 1) MLPSP_SCATTER(1);
    else MLPSP_SCATTER(2);
#undef MLPSP_SCATTER
  } else {
    hipLaunchKernelGGL(bin_level1_kernel, dim3(g.NC, ceil_div(S, kBinThreads / 64)), dim3(kBinThreads), 0, s, b.bounds, g,
                       tile_view_ids_dev, b.l1_counts, b.l1_masks, b.super_view);
  }
  MLPSP_LAUNCH_CHECK();
  hipLaunchKernelGGL(bin_level1_fill_kernel, dim3(S), dim3(kWideThreads), 0, s, b.bounds, g, b.l1_counts, b.l1_list,
                     b.l1_bounds, b.l1_capacity, b.l1_masks, b.super_view, b.l1_super, b.totals, clear_word);
  MLPSP_LAUNCH_CHECK();
  if (!count_tiles) return MLPSP_OK;
  hipLaunchKernelGGL(bin_level2_count_kernel, dim3(level2_groups(T)), dim3(kWideThreads), 0, s, b.bounds, g,
                     tile_view_ids_dev, b.l1_super, b.l1_list, b.l1_bounds, b.l1_capacity, tile_offsets_dev, b.l2_masks,
                     b.l2_mask_stride, b.super_view, b.groups);
  MLPSP_LAUNCH_CHECK();
  if (scan_tiles) {
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(1024), 0, s, tile_offsets_dev, (int)T, b.totals + 1,
                       b.totals + 2);
    MLPSP_LAUNCH_CHECK();
  }
  return MLPSP_OK;
}

// the fill pass of the asynchronous entry points: places the tiles, applies the guard, writes the lists
void enqueue_guarded_fill(const BinGeom& g, const BinScratch& b, int64_t T, const int32_t* tile_view_ids_dev,
                          int32_t* tile_offsets_dev, int32_t* candidates_dev, int64_t cand_capacity, int64_t* counts_dev,
                          hipStream_t s) {
  hipLaunchKernelGGL((bin_level2_fill_kernel<true>), dim3(level2_groups(T)), dim3(kWideThreads), 0, s, g,
                     tile_view_ids_dev, b.l1_super, b.l1_list, b.l1_capacity, tile_offsets_dev, candidates_dev, b.l2_masks,
                     b.l2_mask_stride, b.groups, level2_groups(T),
                     FillGuard{b.totals, (long long*)counts_dev, b.l1_capacity, (long long)cand_capacity});
}

// Enqueues bounds -> level 1 (count, fill) -> level 2 count, no host synchronisation.  With scan_tiles also the
// scan of the tile counts: exclusive tile offsets in tile_offsets_dev and (level-1 entries, pairs, longest tile
// list) in b.totals[0..2].  Without, tile_offsets_dev holds the counts for enqueue_guarded_fill().
int enqueue_bin_count(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                      const float* view_matrices_host, int num_views, const int32_t* tile_view_ids_dev,
                      const float* proj_host, int width, int height, int tile, float threshold, const BinGeom& g,
                      const BinScratch& b, int64_t T, int32_t* tile_offsets_dev, hipStream_t s,
                      bool matrices_in_scratch = false, bool scan_tiles = true, const float* view_dev = nullptr,
                      const float* proj_dev = nullptr, bool count_tiles = true, long long* clear_word = nullptr) {
  BoundsSource src{};
  src.positions = positions_dev;
  src.log_scales = log_scales_dev;
  // scalar constants in f32, in the order the reference's tensor expressions evaluate them
  src.rm = sqrtf(-2.0f * logf(threshold));
  if (view_dev) {             // one view, matrices on the device (the kernel forms the focal length)
    src.mode = 2;
    src.mats = view_dev;
    src.proj_dev = proj_dev;
    return enqueue_bin_levels(src, g, b, T, tile_view_ids_dev, tile_offsets_dev, s, scan_tiles, count_tiles, clear_word);
  }
  const float fx = (proj_host[0] * (float)width) / 2.0f, fy = (proj_host[5] * (float)height) / 2.0f;
  src.focal = (fx + fy) * 0.5f;
  if (num_views == 1) {
    src.mode = 1;
    for (int e = 0; e < 16; ++e) {
      src.one.v[e] = view_matrices_host[e];
      src.one.p[e] = proj_host[e];
    }
  } else {
    src.mode = 0;
    src.mats = b.mats;
    if (!matrices_in_scratch) {
      MLPSP_HIP_TRY(hipMemcpyAsync(b.mats, view_matrices_host, (size_t)num_views * 16 * sizeof(float),
                                   hipMemcpyHostToDevice, s));
      MLPSP_HIP_TRY(hipMemcpyAsync(b.mats + (size_t)num_views * 16, proj_host, 16 * sizeof(float),
                                   hipMemcpyHostToDevice, s));
    }
  }
  return enqueue_bin_levels(src, g, b, T, tile_view_ids_dev, tile_offsets_dev, s, scan_tiles, count_tiles, clear_word);
}

int check_bin_args(int64_t T, const float* view_matrices_host, const float* proj_host, void* scratch_dev,
                   size_t scratch_bytes, int32_t* tile_offsets_dev, int num_primitives, int num_views, int width,
                   int height, int tile, float threshold) {
  if (T <= 0 || num_primitives < 0 || num_views <= 0 || !view_matrices_host || !proj_host || !scratch_dev ||
      !tile_offsets_dev)
    return MLPSP_E_ARGUMENT;
  if (!(threshold > 0.f && threshold < 1.f)) return MLPSP_E_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(tile_offsets_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(scratch_dev) % 256 != 0)
    return MLPSP_E_ARGUMENT;
  if (scratch_bytes < mlpsp_bin_scratch_bytes(num_primitives, num_views, width, height, tile)) return MLPSP_E_SCRATCH;
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_bin_legacy_count(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                                     const float* view_matrices_host, int num_views,
                                     const int32_t* tile_view_ids_dev, const float* proj_host, int width, int height,
                                     int tile, float threshold, void* scratch_dev, size_t scratch_bytes,
                                     int32_t* tile_offsets_dev, int64_t counts_out[2], mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (!counts_out) return MLPSP_E_ARGUMENT;
  const int rc = check_bin_args(T, view_matrices_host, proj_host, scratch_dev, scratch_bytes, tile_offsets_dev,
                                num_primitives, num_views, width, height, tile, threshold);
  if (rc != MLPSP_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  const BinGeom g = make_geom(num_primitives, num_views, width, height, tile);
  const BinScratch b = carve(scratch_dev, scratch_bytes, num_primitives, num_views, g.nsx * g.nsy, g.NC);
  counts_out[0] = counts_out[1] = 0;
  if (num_primitives == 0) {
    MLPSP_HIP_TRY(hipMemsetAsync(tile_offsets_dev, 0, (size_t)(T + 1) * sizeof(int32_t), s));
    MLPSP_HIP_TRY(hipMemsetAsync(b.totals, 0, 4 * sizeof(long long), s));
    return MLPSP_OK;
  }
  const int erc = enqueue_bin_count(positions_dev, log_scales_dev, num_primitives, view_matrices_host, num_views,
                                    tile_view_ids_dev, proj_host, width, height, tile, threshold, g, b, T,
                                    tile_offsets_dev, s);
  if (erc != MLPSP_OK) return erc;
  // one blocking readback: level-1 entry count (overflow check) and the number of pairs
  long long totals[3] = {0, 0, 0};
  MLPSP_HIP_TRY(hipMemcpyAsync(totals, b.totals, 3 * sizeof(long long), hipMemcpyDeviceToHost, s));
  MLPSP_HIP_TRY(hipStreamSynchronize(s));
  if (totals[0] > b.l1_capacity) return MLPSP_E_SCRATCH;
  if (totals[1] > 2147483647LL) return MLPSP_E_ARGUMENT;
  counts_out[0] = totals[1];
  counts_out[1] = totals[2];
  return MLPSP_OK;
}

namespace {
int bin_legacy_async_impl(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                          const float* view_matrices_host, int num_views, const int32_t* tile_view_ids_dev,
                          const float* proj_host, const float* view_dev, const float* proj_dev, int width, int height,
                          int tile, float threshold, void* scratch_dev, size_t scratch_bytes, int32_t* tile_offsets_dev,
                          int32_t* candidates_dev, int64_t cand_capacity, int64_t* counts_dev, hipStream_t s) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (!counts_dev || cand_capacity < 0 || cand_capacity > 2147483647LL || (cand_capacity > 0 && !candidates_dev))
    return MLPSP_E_ARGUMENT;
  // (with device matrices the host pointers stand in for themselves in the argument check: they are not read)
  const float* vh = view_dev ? view_dev : view_matrices_host;
  const float* ph = proj_dev ? proj_dev : proj_host;
  const int rc = check_bin_args(T, vh, ph, scratch_dev, scratch_bytes, tile_offsets_dev, num_primitives, num_views, width,
                                height, tile, threshold);
  if (rc != MLPSP_OK) return rc;
  const BinGeom g = make_geom(num_primitives, num_views, width, height, tile);
  const BinScratch b = carve(scratch_dev, scratch_bytes, num_primitives, num_views, g.nsx * g.nsy, g.NC);
  if (num_primitives == 0) {
    MLPSP_HIP_TRY(hipMemsetAsync(tile_offsets_dev, 0, (size_t)(T + 1) * sizeof(int32_t), s));
    MLPSP_HIP_TRY(hipMemsetAsync(counts_dev, 0, 4 * sizeof(int64_t), s));
    return MLPSP_OK;
  }
  const int erc = enqueue_bin_count(positions_dev, log_scales_dev, num_primitives, view_matrices_host, num_views,
                                    tile_view_ids_dev, proj_host, width, height, tile, threshold, g, b, T,
                                    tile_offsets_dev, s, false, /*scan_tiles=*/false, view_dev, proj_dev);
  if (erc != MLPSP_OK) return erc;
  enqueue_guarded_fill(g, b, T, tile_view_ids_dev, tile_offsets_dev, candidates_dev, cand_capacity, counts_dev, s);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
}  // namespace

MLPSP_API int mlpsp_bin_legacy_async(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                                     const float* view_matrices_host, int num_views,
                                     const int32_t* tile_view_ids_dev, const float* proj_host, int width, int height,
                                     int tile, float threshold, void* scratch_dev, size_t scratch_bytes,
                                     int32_t* tile_offsets_dev, int32_t* candidates_dev, int64_t cand_capacity,
                                     int64_t* counts_dev, mlpsp_stream_t stream) {
  return bin_legacy_async_impl(positions_dev, log_scales_dev, num_primitives, view_matrices_host, num_views,
                               tile_view_ids_dev, proj_host, nullptr, nullptr, width, height, tile, threshold, scratch_dev,
                               scratch_bytes, tile_offsets_dev, candidates_dev, cand_capacity, counts_dev,
                               (hipStream_t)stream);
}

MLPSP_API int mlpsp_bin_legacy_async_device_matrices(const float* positions_dev, const float* log_scales_dev,
                                                     int num_primitives, const float* view_matrix_dev,
                                                     const float* proj_dev, int width, int height, int tile,
                                                     float threshold, void* scratch_dev, size_t scratch_bytes,
                                                     int32_t* tile_offsets_dev, int32_t* candidates_dev,
                                                     int64_t cand_capacity, int64_t* counts_dev,
                                                     mlpsp_stream_t stream) {
  if (!view_matrix_dev || !proj_dev) return MLPSP_E_ARGUMENT;
  return bin_legacy_async_impl(positions_dev, log_scales_dev, num_primitives, nullptr, 1, nullptr, nullptr, view_matrix_dev,
                               proj_dev, width, height, tile, threshold, scratch_dev, scratch_bytes, tile_offsets_dev,
                               candidates_dev, cand_capacity, counts_dev, (hipStream_t)stream);
}

MLPSP_API int mlpsp_bin_segments_async_device_matrices(const float* positions_dev, const float* log_scales_dev,
                                                       int num_primitives, const float* view_matrix_dev,
                                                       const float* proj_dev, int width, int height, int tile,
                                                       float threshold, void* scratch_dev, size_t scratch_bytes,
                                                       int segment_stride, int32_t* tile_offsets_dev,
                                                       int32_t* tile_ends_dev, int32_t* candidates_dev,
                                                       int64_t* counts_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (!view_matrix_dev || !proj_dev || !counts_dev || !tile_ends_dev || !candidates_dev || segment_stride <= 0)
    return MLPSP_E_ARGUMENT;
  const int rc = check_bin_args(T, view_matrix_dev, proj_dev, scratch_dev, scratch_bytes, tile_offsets_dev,
                                num_primitives, 1, width, height, tile, threshold);
  if (rc != MLPSP_OK) return rc;
  if (T > 2147483647LL / segment_stride) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  const BinGeom g = make_geom(num_primitives, 1, width, height, tile);
  const BinScratch b = carve(scratch_dev, scratch_bytes, num_primitives, 1, g.nsx * g.nsy, g.NC);
  if (num_primitives == 0) {        // every list empty: [0, 0)
    MLPSP_HIP_TRY(hipMemsetAsync(tile_offsets_dev, 0, (size_t)(T + 1) * sizeof(int32_t), s));
    MLPSP_HIP_TRY(hipMemsetAsync(tile_ends_dev, 0, (size_t)T * sizeof(int32_t), s));
    MLPSP_HIP_TRY(hipMemsetAsync(counts_dev, 0, 4 * sizeof(int64_t), s));
    return MLPSP_OK;
  }
  const int erc = enqueue_bin_count(positions_dev, log_scales_dev, num_primitives, nullptr, 1, nullptr, nullptr, width,
                                    height, tile, threshold, g, b, T, tile_offsets_dev, s, false, /*scan_tiles=*/false,
                                    view_matrix_dev, proj_dev, /*count_tiles=*/false,
                                    reinterpret_cast<long long*>(counts_dev) + 1);
  if (erc != MLPSP_OK) return erc;
  hipLaunchKernelGGL(bin_level2_segments_kernel, dim3(level2_groups(T)), dim3(kWideThreads), 0, s, b.bounds, g,
                     (const int32_t*)nullptr, b.l1_super, b.l1_list, b.l1_bounds, b.l1_capacity, b.l2_masks,
                     b.l2_mask_stride, b.super_view, b.totals, segment_stride, tile_offsets_dev, tile_ends_dev,
                     candidates_dev, reinterpret_cast<long long*>(counts_dev));
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_bin_legacy_fill(int num_primitives, int num_views, const int32_t* tile_view_ids_dev, int width,
                                    int height, int tile, const void* scratch_dev, size_t scratch_bytes,
                                    const int32_t* tile_offsets_dev, int32_t* candidates_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (T <= 0 || num_primitives < 0 || num_views <= 0 || !scratch_dev || !tile_offsets_dev) return MLPSP_E_ARGUMENT;
  if (num_primitives == 0) return MLPSP_OK;
  if (!candidates_dev) return MLPSP_E_ARGUMENT;
  const BinGeom g = make_geom(num_primitives, num_views, width, height, tile);
  const BinScratch b = carve(const_cast<void*>(scratch_dev), scratch_bytes, num_primitives, num_views, g.nsx * g.nsy, g.NC);
  hipLaunchKernelGGL((bin_level2_fill_kernel<false>), dim3(level2_groups(T)), dim3(kWideThreads), 0, (hipStream_t)stream,
                     g, tile_view_ids_dev, b.l1_super, b.l1_list, b.l1_capacity, const_cast<int32_t*>(tile_offsets_dev),
                     candidates_dev, b.l2_masks, b.l2_mask_stride, b.groups, level2_groups(T),
                     FillGuard{nullptr, nullptr, 0, 0});
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

// ---------------------------------------------------------------------------------------------
// The asynchronous binning for callers that cannot allocate: its scratch is a file-scope device array.
// ---------------------------------------------------------------------------------------------
namespace mlpsp {
constexpr size_t kStaticBinScratchBytes = MLPSP_BIN_STATIC_SCRATCH_BYTES;
constexpr int kStaticBinMaxViews = MLPSP_BIN_STATIC_MAX_VIEWS;
static __device__ __align__(256) unsigned char scratch[kStaticBinScratchBytes];

struct ManyMats {
  float v[kStaticBinMaxViews][16];
  float p[16];
};
// view and projection matrices travel as kernel arguments and are stored where the binning kernels read them
__global__ __launch_bounds__(64) void store_matrices_kernel(ManyMats m, int num_views, float* __restrict__ dst) {
  const int t = threadIdx.x;
  if (t < 16) {
    for (int k = 0; k < num_views; ++k) dst[k * 16 + t] = m.v[k][t];
    dst[num_views * 16 + t] = m.p[t];
  }
}
__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* __restrict__ dst, long long n, int32_t value) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
    dst[i] = value;
}
}  // namespace mlpsp

namespace {
// address of the array on each device, taken once per device with that device current
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices];
bool g_static_scratch_known[kMaxDevices];

int static_scratch_of_current_device(void** out) {
  int dev = -1;
  MLPSP_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return MLPSP_E_ARGUMENT;
  // (two threads racing here both obtain the same address; the flag is written last)
  if (!__atomic_load_n(&g_static_scratch_known[dev], __ATOMIC_ACQUIRE)) {
    void* ptr = nullptr;
    MLPSP_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(mlpsp::scratch)));
    if (!ptr) return MLPSP_E_RUNTIME;
    g_static_scratch[dev] = ptr;
    __atomic_store_n(&g_static_scratch_known[dev], true, __ATOMIC_RELEASE);
  }
  *out = g_static_scratch[dev];
  return MLPSP_OK;
}
}  // namespace

MLPSP_API size_t mlpsp_bin_static_scratch_bytes(void) { return kStaticBinScratchBytes; }

MLPSP_API int mlpsp_bin_legacy_async_noalloc(const float* positions_dev, const float* log_scales_dev,
                                             int num_primitives, const float* view_matrices_host, int num_views,
                                             const int32_t* tile_view_ids_dev, const float* proj_host, int width,
                                             int height, int tile, float threshold, int32_t* tile_offsets_dev,
                                             int32_t* candidates_dev, int64_t cand_capacity, int64_t* counts_dev,
                                             mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (!counts_dev || cand_capacity < 0 || cand_capacity > 2147483647LL || (cand_capacity > 0 && !candidates_dev))
    return MLPSP_E_ARGUMENT;
  if (num_views > kStaticBinMaxViews) return MLPSP_E_ARGUMENT;
  void* scratch_dev = nullptr;
  const int src = static_scratch_of_current_device(&scratch_dev);
  if (src != MLPSP_OK) return src;
  const size_t need = mlpsp_bin_scratch_bytes(num_primitives, num_views, width, height, tile);
  if (need == 0) return MLPSP_E_ARGUMENT;
  if (need > kStaticBinScratchBytes) return MLPSP_E_SCRATCH;      // beyond the fixed maximum: use mlpsp_bin_legacy_async
  const int rc = check_bin_args(T, view_matrices_host, proj_host, scratch_dev, kStaticBinScratchBytes, tile_offsets_dev,
                                num_primitives, num_views, width, height, tile, threshold);
  if (rc != MLPSP_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  const BinGeom g = make_geom(num_primitives, num_views, width, height, tile);
  // The whole array is carved, not just the bytes the ordinary entry point asks for: what is left over goes to the
  // level-1 lists, whose overflow (guard word raised, lists emptied) a caller that cannot allocate could not answer
  // with a larger scratch.  Lists do not depend on the capacity they were built in: same outputs as
  // mlpsp_bin_legacy_async wherever that one does not overflow.
  const BinScratch b = carve(scratch_dev, kStaticBinScratchBytes, num_primitives, num_views, g.nsx * g.nsy, g.NC);
  if (num_primitives == 0) {
    hipLaunchKernelGGL(fill_i32_kernel, dim3(64), dim3(256), 0, s, tile_offsets_dev, (long long)(T + 1), 0);
    MLPSP_LAUNCH_CHECK();
    hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<int32_t*>(counts_dev), 8LL, 0);
    MLPSP_LAUNCH_CHECK();
    return MLPSP_OK;
  }
  if (num_views > 1) {
    ManyMats m{};
    for (int k = 0; k < num_views; ++k)
      for (int e = 0; e < 16; ++e) m.v[k][e] = view_matrices_host[k * 16 + e];
    for (int e = 0; e < 16; ++e) m.p[e] = proj_host[e];
    hipLaunchKernelGGL(store_matrices_kernel, dim3(1), dim3(64), 0, s, m, num_views, b.mats);
    MLPSP_LAUNCH_CHECK();
  }
  const int erc = enqueue_bin_count(positions_dev, log_scales_dev, num_primitives, view_matrices_host, num_views,
                                    tile_view_ids_dev, proj_host, width, height, tile, threshold, g, b, T,
                                    tile_offsets_dev, s, /*matrices_in_scratch=*/true, /*scan_tiles=*/false);
  if (erc != MLPSP_OK) return erc;
  enqueue_guarded_fill(g, b, T, tile_view_ids_dev, tile_offsets_dev, candidates_dev, cand_capacity, counts_dev, s);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
