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
  int cnt[kSortThreads], off[kSortThreads];
  uint16_t perm[kSortMax], order[kSortMax];
  uint32_t kmin, kmax;
  int flags, pairs;
};

// Per-frame, per-primitive record of the sort (64 bytes, one cache line per candidate): what the key and the culling
// test need of a primitive once the ray origin is known.  Whenever the rays of a frame start from one point (a
// pinhole camera: always) the rotated offset vl = R(q)^T (c - o) of the key (np_tile_kernels.cu:483-500) depends on
// the primitive alone; frame_sort_records_kernel evaluates it once per primitive with the very expressions of
// key_tstar(), so the key of a candidate costs one quaternion rotation (the ray direction's) instead of two, with
// the same bits.  For the culling test the record carries e = c - o and the world-space covariance
// S = R diag(s^2) R^T, so that the support of the threshold ellipsoid along a face normal n is the quadratic form
// n^T S n (six multiply-adds against per-tile products of the normal) instead of a rotation of n per face.  S is
// stored as six bf16 values rounded so that the stored matrix minus the exact one is positive semi-definite
// (off-diagonal entries to nearest, every diagonal entry raised by its row's rounding errors plus 1e-5 of the
// trace, then rounded up): the quadratic form never comes out smaller than the exact one, i.e. the test stays
// conservative, at a few percent of the smallest axis for ordinary shapes.
struct __attribute__((aligned(64))) SortRec {
  float qw, qx, qy, qz;
  float mx, my, mz, vlx;
  float vly, vlz, ex, ey;
  float ez;
  uint32_t s_xx_yy, s_zz_xy, s_xz_yz;      // (first << 16 | second), each the upper half of an f32
};
static_assert(sizeof(SortRec) == MLPSP_SORT_RECORD_BYTES, "record size is part of the C ABI");
// Slot 0 of the record buffer: the origin the records were made for (its bits) and whether they were made at all.
struct __attribute__((aligned(64))) SortFrameHeader {
  uint32_t ox, oy, oz;
  int32_t valid;
  uint32_t pad[12];
};
static_assert(sizeof(SortFrameHeader) == sizeof(SortRec), "the header takes one record slot");

__device__ __forceinline__ uint32_t bf16_nearest(float x) {     // upper 16 bits, round to nearest even
  const uint32_t u = float_to_bits(x);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ uint32_t bf16_up(float x) {          // x >= 0: the smallest bf16 at or above x
  const uint32_t u = float_to_bits(x);
  return (u >> 16) + ((u & 0xffffu) ? 1u : 0u);
}

// The record of primitive p (thread p = 0 also writes the header).  origin = rays_o[0..2].
__device__ __forceinline__ void write_frame_sort_record(const float* __restrict__ rays_o,
                                                        const PrimRecord* __restrict__ prims, int N,
                                                        SortRec* __restrict__ out, int p) {
  const float ox = rays_o[0], oy = rays_o[1], oz = rays_o[2];
  if (p == 0) {
    SortFrameHeader h = {};
    h.ox = float_to_bits(ox);
    h.oy = float_to_bits(oy);
    h.oz = float_to_bits(oz);
    h.valid = 1;
    *reinterpret_cast<SortFrameHeader*>(out) = h;
  }
  if (p >= N) return;
  const float4* src = reinterpret_cast<const float4*>(prims + p);
  const float4 a = src[0], b = src[1], c = src[2], d = src[3];
  PrimRecord P;
  P.cx = a.x; P.cy = a.y; P.cz = a.z; P.mx = a.w;
  P.my = b.x; P.mz = b.y; P.qw = b.z; P.qx = b.w;
  P.qy = c.x; P.qz = c.y;
  P.s2x = d.y; P.s2y = d.z; P.s2z = d.w;
  // exactly the first statements of key_tstar()
  const Vec3 v = {P.cx - ox, P.cy - oy, P.cz - oz};
  const Vec3 vl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, v);
  // covariance in world axes: columns of R(q) are the ellipsoid's axes
  const float w = P.qw, x = P.qx, y = P.qy, z = P.qz;
  const float r00 = 1.f - 2.f * (y * y + z * z), r01 = 2.f * (x * y - w * z), r02 = 2.f * (x * z + w * y);
  const float r10 = 2.f * (x * y + w * z), r11 = 1.f - 2.f * (x * x + z * z), r12 = 2.f * (y * z - w * x);
  const float r20 = 2.f * (x * z - w * y), r21 = 2.f * (y * z + w * x), r22 = 1.f - 2.f * (x * x + y * y);
  const float sx = P.s2x, sy = P.s2y, sz = P.s2z;
  const float cxx = fmaf(sx, r00 * r00, fmaf(sy, r01 * r01, sz * (r02 * r02)));
  const float cyy = fmaf(sx, r10 * r10, fmaf(sy, r11 * r11, sz * (r12 * r12)));
  const float czz = fmaf(sx, r20 * r20, fmaf(sy, r21 * r21, sz * (r22 * r22)));
  const float cxy = fmaf(sx, r00 * r10, fmaf(sy, r01 * r11, sz * (r02 * r12)));
  const float cxz = fmaf(sx, r00 * r20, fmaf(sy, r01 * r21, sz * (r02 * r22)));
  const float cyz = fmaf(sx, r10 * r20, fmaf(sy, r11 * r21, sz * (r12 * r22)));
  const uint32_t hxy = bf16_nearest(cxy), hxz = bf16_nearest(cxz), hyz = bf16_nearest(cyz);
  const float exy = fabsf(cxy - bits_to_float(hxy << 16)), exz = fabsf(cxz - bits_to_float(hxz << 16)),
              eyz = fabsf(cyz - bits_to_float(hyz << 16));
  const float slack = 1e-5f * ((cxx + cyy) + czz);
  const uint32_t hxx = bf16_up((cxx + slack) + (exy + exz)), hyy = bf16_up((cyy + slack) + (exy + eyz)),
                 hzz = bf16_up((czz + slack) + (exz + eyz));
  float4* dst = reinterpret_cast<float4*>(out + 1 + p);
  dst[0] = make_float4(P.qw, P.qx, P.qy, P.qz);
  dst[1] = make_float4(P.mx, P.my, P.mz, vl.x);
  dst[2] = make_float4(vl.y, vl.z, v.x, v.y);
  dst[3] = make_float4(v.z, bits_to_float((hxx << 16) | (hyy & 0xffffu)), bits_to_float((hzz << 16) | (hxy & 0xffffu)),
                       bits_to_float((hxz << 16) | (hyz & 0xffffu)));
}
// One thread per primitive.
__global__ __launch_bounds__(256) void frame_sort_records_kernel(const float* __restrict__ rays_o,
                                                                 const PrimRecord* __restrict__ prims, int N,
                                                                 SortRec* __restrict__ out) {
  write_frame_sort_record(rays_o, prims, N, out, blockIdx.x * blockDim.x + threadIdx.x);
}

// key_tstar() with vl taken from the frame record: the remaining statements, unchanged.
__device__ __forceinline__ float key_tstar_hoisted(float dx, float dy, float dz, const SortRec& R) {
  const Vec3 vl = {R.vlx, R.vly, R.vlz};
  const Vec3 dl = quat_rotate_conj(R.qw, R.qx, R.qy, R.qz, Vec3{dx, dy, dz});
  const float denom = fmaf(dl.x * dl.x, R.mx, fmaf(dl.y * dl.y, R.my, (dl.z * dl.z) * R.mz));
  const float numer = fmaf(dl.x * vl.x, R.mx, fmaf(dl.y * vl.y, R.my, (dl.z * vl.z) * R.mz));
  const float t = numer / denom;
  return (denom > 1e-20f && t > 0.f) ? t : kInvalidKey;
}
// key_depth() with c - o taken from the frame record.
__device__ __forceinline__ float key_depth_hoisted(float dx, float dy, float dz, const SortRec& R) {
  const float k = fmaf(R.ex, dx, fmaf(R.ey, dy, R.ez * dz));
  return (k > 0.f) ? k : kInvalidKey;
}

// The pyramid of a tile's rays: four planes through the common origin, each spanned by two neighbouring corner
// rays and oriented towards the tile-centre ray.  Everything in it is the same for every lane (it is read out of
// the lanes that computed it with v_readlane), so the per-candidate tests take it as scalar operands.
struct TilePyramid {
  float ox, oy, oz;        // the tile's common origin (corner 0's)
  float n[4][3];           // inward normals
  float q[4][6];           // nx^2, ny^2, nz^2, 2 nx ny, 2 nx nz, 2 ny nz of each
  int faces;               // bit j: face j may be used (0: no culling for this tile)
};
__device__ __forceinline__ float lane_value(float v, int lane) {
  return bits_to_float((uint32_t)__builtin_amdgcn_readlane((int)float_to_bits(v), lane));
}
// How tile_pyramid() reads the direction of a pixel's ray: unit vectors as stored, or directions as the caller
// holds them, normalised on the way (the frame prologue runs beside the kernel that writes the unit vectors).  The
// pyramid only needs directions of about unit length, so that its tolerances mean what they say: a reciprocal square
// root and three products, not the exactly rounded square root and divisions of the unit vectors the renderer uses
// (four of those per lane were three quarters of the prologue's pyramid work).  The planes then differ from those
// built from the stored unit vectors in their last bits; the culling has a 2 % margin either way.
struct UnitDirs {
  const float* __restrict__ d;
  __device__ __forceinline__ void get(int pix, float& x, float& y, float& z) const {
    const Float3 v = load3(d, pix);
    x = v.x;
    y = v.y;
    z = v.z;
  }
};
struct RawDirs {
  const float* __restrict__ d;
  __device__ __forceinline__ void get(int pix, float& x, float& y, float& z) const {
    const Float3 v = load3(d, pix);
    const float r = __builtin_amdgcn_rsqf(fmaxf((v.x * v.x + v.z * v.z) + v.y * v.y, 1e-24f));
    x = v.x * r;
    y = v.y * r;
    z = v.z * r;
  }
};

// Called by a whole wavefront: lane l builds face l % 4 (face j from corner rays j and j + 1), then every lane
// checks rays of the tile (all of them between the 64 lanes) against the four faces and the common origin.  A face
// the centre ray (nearly) lies in, or that some ray of the tile is outside of, is not used; without a common origin
// none is.  The roundings here are free: the per-candidate test has a 2 % margin.
template <typename Dirs>
__device__ __forceinline__ TilePyramid tile_pyramid(const float* __restrict__ rays_o, const Dirs dirs,
                                                    const TileGeom& g, int tile, float dx, float dy, float dz) {
  const int lane = threadIdx.x & 63;
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int x0 = tx * g.TW, y0 = ty * g.TH;
  const int x1 = min(x0 + g.TW, g.W) - 1, y1 = min(y0 + g.TH, g.H) - 1;
  const int j = lane & 3, j1 = (lane + 1) & 3;
  // corners in the order (x0,y0) (x1,y0) (x1,y1) (x0,y1)
  const int ca = ((j >> 1) ? y1 : y0) * g.W + ((j == 1 || j == 2) ? x1 : x0);
  const int cb = ((j1 >> 1) ? y1 : y0) * g.W + ((j1 == 1 || j1 == 2) ? x1 : x0);
  float a0, a1, a2, b0, b1, b2;
  dirs.get(ca, a0, a1, a2);
  dirs.get(cb, b0, b1, b2);
  const int c0 = y0 * g.W + x0;
  TilePyramid py;
  const Float3 origin = load3(rays_o, c0);
  py.ox = origin.x;
  py.oy = origin.y;
  py.oz = origin.z;
  float nx = a1 * b2 - a2 * b1, ny = a2 * b0 - a0 * b2, nz = a0 * b1 - a1 * b0;
  const float side = nx * dx + ny * dy + nz * dz;
  const float len = __builtin_amdgcn_sqrtf(nx * nx + ny * ny + nz * nz);
  const bool usable = len > 0.f && fabsf(side) > 1e-4f * len;
  const float sgn = side < 0.f ? -1.f : 1.f;
  nx *= sgn;
  ny *= sgn;
  nz *= sgn;
  const float prod[6] = {nx * nx, ny * ny, nz * nz, 2.f * (nx * ny), 2.f * (nx * nz), 2.f * (ny * nz)};
  float nlen[4];
  int ok = 0x10;
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    py.n[f][0] = lane_value(nx, f);
    py.n[f][1] = lane_value(ny, f);
    py.n[f][2] = lane_value(nz, f);
    nlen[f] = lane_value(len, f);
#pragma unroll
    for (int k = 0; k < 6; ++k) py.q[f][k] = lane_value(prod[k], f);
    ok |= ((__ballot(usable) >> f) & 1ull) ? (1 << f) : 0;
  }
  for (int k = lane; k < g.TW * g.TH; k += 64) {
    const int x = x0 + k % g.TW, y = y0 + k / g.TW;
    if (x < g.W && y < g.H) {
      const int pix = y * g.W + x;
      const Float3 o = load3(rays_o, pix);
      if (o.x != py.ox || o.y != py.oy || o.z != py.oz) ok &= ~0x10;
      float rx, ry, rz;
      dirs.get(pix, rx, ry, rz);
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const float inside = py.n[f][0] * rx + py.n[f][1] * ry + py.n[f][2] * rz;
        if (!(inside >= -1e-6f * nlen[f])) ok &= ~(1 << f);
      }
    }
  }
  int all_ok = 0;
#pragma unroll
  for (int b = 0; b < 5; ++b) all_ok |= __ballot(!((ok >> b) & 1)) ? 0 : (1 << b);
  py.faces = (all_ok & 0x10) ? (all_ok & 0xf) : 0;
  return py;
}

// The pyramid of a tile as the frame prologue leaves it for the sort: the four normals, the origin, the usable
// faces, the products of the normals' components (forty words).  Built once per tile there; a sort that is not handed such records builds the pyramid in each of a tile's
// wavefronts, whose strided reads of the tile's 64 rays (12-byte stride over eight image rows, by all four
// wavefronts) measured 18 us of the 134 us launch at 12,750 tiles.
struct alignas(32) TilePyramidRec {
  float n[4][3];
  float ox, oy, oz;
  int faces;
  float q[4][6];
};
static_assert(sizeof(TilePyramidRec) == MLPSP_TILE_PYRAMID_BYTES && MLPSP_TILE_PYRAMID_BYTES == 40 * 4,
              "forty words per tile");
// One wavefront per tile; `raw` are the directions before normalisation.
__device__ __forceinline__ void write_tile_pyramid(const float* __restrict__ rays_o, const float* __restrict__ raw,
                                                   const TileGeom& g, int tile, TilePyramidRec* __restrict__ out) {
  const int pc = centre_pixel(g, tile);
  float dx, dy, dz;
  RawDirs{raw}.get(pc, dx, dy, dz);
  const TilePyramid py = tile_pyramid(rays_o, RawDirs{raw}, g, tile, dx, dy, dz);
  if ((threadIdx.x & 63) == 0) {
    TilePyramidRec r;
#pragma unroll
    for (int f = 0; f < 4; ++f) {
#pragma unroll
      for (int k = 0; k < 3; ++k) r.n[f][k] = py.n[f][k];
#pragma unroll
      for (int k = 0; k < 6; ++k) r.q[f][k] = py.q[f][k];
    }
    r.ox = py.ox;
    r.oy = py.oy;
    r.oz = py.oz;
    r.faces = py.faces;
    out[tile] = r;
  }
}
// A record as a wavefront holds it: lane j has word j (one coalesced load), and the words are taken out of that
// register with v_readlane, the way tile_pyramid() hands out what its lanes computed.
__device__ __forceinline__ float pyramid_record_word(const TilePyramidRec* __restrict__ record) {
  const int lane = threadIdx.x & 63;
  return reinterpret_cast<const float*>(record)[lane < 40 ? lane : 0];
}
__device__ __forceinline__ TilePyramid pyramid_from_word(float word) {
  TilePyramid py;
  py.ox = lane_value(word, 12);
  py.oy = lane_value(word, 13);
  py.oz = lane_value(word, 14);
  py.faces = (int)float_to_bits(lane_value(word, 15));
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    const float nx = lane_value(word, f * 3), ny = lane_value(word, f * 3 + 1), nz = lane_value(word, f * 3 + 2);
    py.n[f][0] = nx;
    py.n[f][1] = ny;
    py.n[f][2] = nz;
#pragma unroll
    for (int k = 0; k < 6; ++k) py.q[f][k] = lane_value(word, 16 + f * 6 + k);
  }
  return py;
}

// Can no ray of the tile hit the primitive?  True if its threshold ellipsoid lies wholly beyond one usable face.
// General form: every face normal is taken into the primitive's axes with the rotation matrix of the quaternion,
// worked out once per candidate (24 instructions + 9 per face, where a quaternion rotation per face costs 21; fused
// multiply-adds throughout: roundings are free here, the test keeps a margin of 2 % of the radius).
__device__ __forceinline__ bool outside_pyramid(const TilePyramid& py, const PrimRecord& P, float cull_r2) {
  bool outside = false;
  const float ex = P.cx - py.ox, ey = P.cy - py.oy, ez = P.cz - py.oz;
  // R(q), local -> world; a normal goes world -> local with its transpose
  const float w = P.qw, x = P.qx, y = P.qy, z = P.qz;
  const float x2 = x + x, y2 = y + y, z2 = z + z;
  const float xx = x * x2, yy = y * y2, zz = z * z2, xy = x * y2, xz = x * z2, yz = y * z2;
  const float wx = w * x2, wy = w * y2, wz = w * z2;
  const float r00 = 1.f - (yy + zz), r01 = xy - wz, r02 = xz + wy;
  const float r10 = xy + wz, r11 = 1.f - (xx + zz), r12 = yz - wx;
  const float r20 = xz - wy, r21 = yz + wx, r22 = 1.f - (xx + yy);
  // squared semi-axes as reciprocals of the precision diagonal (one unit in the last place, far inside the margin;
  // 1/0 = inf never culls): the record's own s2 words lie in its fourth 16-byte piece, which nothing else here
  // needs -- a candidate is then three requests instead of four
  // (with the squared cull radius folded in: beyond a face means dist < 0 and dist^2 > r^2 h^2, i.e.
  // dist |dist| < -(r^2 h^2): one product and one comparison per face)
  const float s2x = cull_r2 * __builtin_amdgcn_rcpf(P.mx), s2y = cull_r2 * __builtin_amdgcn_rcpf(P.my),
              s2z = cull_r2 * __builtin_amdgcn_rcpf(P.mz);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float nx = py.n[j][0], ny = py.n[j][1], nz = py.n[j][2];
    const float dist = fmaf(nx, ex, fmaf(ny, ey, nz * ez));
    const float lx = fmaf(r00, nx, fmaf(r10, ny, r20 * nz));
    const float ly = fmaf(r01, nx, fmaf(r11, ny, r21 * nz));
    const float lz = fmaf(r02, nx, fmaf(r12, ny, r22 * nz));
    const float h2 = fmaf(s2x * lx, lx, fmaf(s2y * ly, ly, (s2z * lz) * lz));
    outside |= ((py.faces >> j) & 1) && (dist * __builtin_fabsf(dist) < -h2);
  }
  return outside;
}
// With a frame record: the support along n is the quadratic form of the (conservatively rounded) covariance.
__device__ __forceinline__ bool outside_pyramid(const TilePyramid& py, const SortRec& R, float cull_r2) {
  bool outside = false;
  const float sxx = bits_to_float(R.s_xx_yy & 0xffff0000u), syy = bits_to_float(R.s_xx_yy << 16);
  const float szz = bits_to_float(R.s_zz_xy & 0xffff0000u), sxy = bits_to_float(R.s_zz_xy << 16);
  const float sxz = bits_to_float(R.s_xz_yz & 0xffff0000u), syz = bits_to_float(R.s_xz_yz << 16);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float dist = fmaf(py.n[j][0], R.ex, fmaf(py.n[j][1], R.ey, py.n[j][2] * R.ez));
    const float h2 = fmaf(py.q[j][0], sxx, fmaf(py.q[j][1], syy, fmaf(py.q[j][2], szz,
                     fmaf(py.q[j][3], sxy, fmaf(py.q[j][4], sxz, py.q[j][5] * syz)))));
    outside |= ((py.faces >> j) & 1) && (dist < 0.f) && (dist * dist >= cull_r2 * h2);
  }
  return outside;
}

// The two sources of a candidate's geometry as one interface: keep-or-cull, and the key.
struct FromPrimRecord {
  typedef PrimRecord Rec;
  const PrimRecord* __restrict__ base;
  float ox, oy, oz;                         // origin of the tile-centre ray
  __device__ __forceinline__ Rec load(int p) const {
    // (only the first 64 bytes are used below: the compiler requests no more)
    return base[p];
  }
  __device__ __forceinline__ float key(int family, float dx, float dy, float dz, const Rec& P) const {
    return (family == MLPSP_KEY_DEPTH) ? key_depth(ox, oy, oz, dx, dy, dz, P) : key_tstar(ox, oy, oz, dx, dy, dz, P);
  }
};
struct FromFrameRecord {
  typedef SortRec Rec;
  const SortRec* __restrict__ base;         // record of primitive 0
  __device__ __forceinline__ Rec load(int p) const {
    return base[p];
  }
  __device__ __forceinline__ float key(int family, float dx, float dy, float dz, const Rec& R) const {
    return (family == MLPSP_KEY_DEPTH) ? key_depth_hoisted(dx, dy, dz, R) : key_tstar_hoisted(dx, dy, dz, R);
  }
};
// Do the frame records (if any) hold for a tile whose centre ray starts at (ox, oy, oz)?
__device__ __forceinline__ bool frame_records_hold(const SortRec* __restrict__ frame, float ox, float oy, float oz) {
  if (!frame) return false;
  const SortFrameHeader& h = *reinterpret_cast<const SortFrameHeader*>(frame);
  return h.valid == 1 && h.ox == float_to_bits(ox) && h.oy == float_to_bits(oy) && h.oz == float_to_bits(oz);
}

// A tile whose list has at most 64 entries, sorted by ONE wavefront (lane = entry) in registers: no LDS, no barrier.
// Same output as sort_one_tile() -- the kept entries ordered by their (key bits, list position) words, which also
// puts keys at or above the invalid key last and in list order among equals; culled entries as ~id at the end of
// the tile's output, last one first -- at a fifth of its instructions: for short lists sort_one_tile()'s cost is
// what four wavefronts spend per tile whatever its length (the passes of the bucket ranking, a dozen barriers).
// Requires len <= 64 and len <= capacity; called by a whole wavefront.
template <bool PYR, typename Source>
__device__ __forceinline__ void sort_small_tile_from(
    const Source& src, const float* __restrict__ rays_o, const float* __restrict__ rays_d,
    const TilePyramidRec* __restrict__ pyramids, const TileGeom& g, int tile, float dx, float dy, float dz,
    const int32_t* __restrict__ cand, int family, float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids,
    float* __restrict__ sorted_keys, int start, int n) {
  const int lane = threadIdx.x & 63;
  const int p = (lane < n) ? cand[start + lane] : 0;
  const bool known = (unsigned)p < (unsigned)num_prims;
  const typename Source::Rec P = src.load(known ? p : 0);
  TilePyramid py = {};
  if (cull_r2 > 0.f) {
    if constexpr (PYR) py = pyramid_from_word(pyramid_record_word(pyramids + tile));
    else py = tile_pyramid(rays_o, UnitDirs{rays_d}, g, tile, dx, dy, dz);
  }
  bool keep = false;
  float key = 0.f;
  if (lane < n) {
    keep = !(py.faces && known && outside_pyramid(py, P, cull_r2));
    if (keep) key = !known ? kInvalidKey : src.key(family, dx, dy, dz, P);
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
template <bool PYR>
__device__ __forceinline__ void sort_small_tile(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const SortRec* __restrict__ frame, const TilePyramidRec* __restrict__ pyramids, const int32_t* __restrict__ cand,
    const TileGeom& g, int family, float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids,
    float* __restrict__ sorted_keys, int tile, int start, int n) {
  const int pc = centre_pixel(g, tile);
  const float ox = rays_o[pc * 3 + 0], oy = rays_o[pc * 3 + 1], oz = rays_o[pc * 3 + 2];
  const float dx = rays_d[pc * 3 + 0], dy = rays_d[pc * 3 + 1], dz = rays_d[pc * 3 + 2];
  if (frame_records_hold(frame, ox, oy, oz))
    sort_small_tile_from<PYR>(FromFrameRecord{frame + 1}, rays_o, rays_d, pyramids, g, tile, dx, dy, dz, cand, family,
                         cull_r2, num_prims, sorted_ids, sorted_keys, start, n);
  else
    sort_small_tile_from<PYR>(FromPrimRecord{prims, ox, oy, oz}, rays_o, rays_d, pyramids, g, tile, dx, dy, dz, cand, family,
                         cull_r2, num_prims, sorted_ids, sorted_keys, start, n);
}

// Sorts one tile with the calling 256-thread workgroup (every thread must call it; `tile` is uniform).  kSortMax
// bounds `capacity`.  A workgroup that sorts several tiles in a row, or uses `lds` for something else afterwards,
// puts a barrier in between.
// ASC: the caller vouches that the list's ids ascend (the own binning writes them so).  Then (key, id) orders like
// (key, list position), the word that is sorted carries the id itself, and the output needs no second look at the
// list.
template <int kSortMax, bool PYR, bool ASC, typename Source>
__device__ __forceinline__ void sort_one_tile_from(SortLds<kSortMax>& lds, const Source& src,
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const TilePyramidRec* __restrict__ pyramids,
    const TileGeom& g, int tile, float dx, float dy, float dz, const int32_t* __restrict__ cand, int family,
    float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids, float* __restrict__ sorted_keys, int start, int len,
    int n) {
  auto& s_key = lds.key;
  auto& s_wave_cnt = lds.wave_cnt;
  auto& s_cnt = lds.cnt;
  auto& s_off = lds.off;
  auto& s_perm = lds.perm;
  auto& s_order = lds.order;
  auto& s_kmin = lds.kmin;
  auto& s_kmax = lds.kmax;
  auto& s_flags = lds.flags;
  auto& s_pairs = lds.pairs;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // (the wavefront's index as a scalar)

  // Every candidate id this thread will handle is requested up front (at most kSortMax / kSortThreads of them),
  // and the first round's geometry record right behind; each round of the key loop then requests the next round's
  // record.  An id outside [0, num_prims) (lists that were never validated) reads record 0, is never culled and
  // sorts last with the invalid key; it is passed on unchanged, and the render kernels skip it.
  constexpr int kRounds = kSortMax / kSortThreads;
  int my_id[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) my_id[r] = (tid + r * kSortThreads < n) ? cand[start + tid + r * kSortThreads] : 0;
  typename Source::Rec P_buf[2];                         // this round's record and the next round's
  P_buf[0] = src.load(((unsigned)my_id[0] < (unsigned)num_prims) ? my_id[0] : 0);

  // ---- the tile's ray pyramid (only when culling is requested), while those loads are on their way: every
  //      wavefront builds it for itself -- four faces among its lanes, one ray of the tile per lane -- so no barrier
  //      is needed for the verdict
  // (PYR is a compile-time choice: with both forms behind one run-time branch, or with the record read as sixteen
  // scalar words, the compiler keeps the pyramid in vector registers for the candidate loop -- 96 registers instead of
  // 72 and a wavefront less per SIMD.  A record therefore arrives in ONE vector register, a word per lane, and the
  // sixteen words the face test needs are taken out of it with v_readlane: they are scalar operands of its
  // multiply-adds and stay in scalar registers over the rounds.)
  TilePyramid py = {};
  float pyramid_word = 0.f;
  int faces = 0;
  if (cull_r2 > 0.f) {
    if constexpr (PYR) {
      pyramid_word = pyramid_record_word(pyramids + tile);
      faces = (int)float_to_bits(lane_value(pyramid_word, 15));
    } else {
      py = tile_pyramid(rays_o, UnitDirs{rays_d}, g, tile, dx, dy, dz);
      faces = py.faces;
    }
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
  // ordinary survivors so far in the low half, late ones in the high half (block-uniform; a list holds at most
  // kSortMax <= 65,535 entries, so the halves never carry into each other): one sum serves both streams
  int survivors = 0;
  uint32_t key_lo = 0xffffffffu, key_hi = 0u;
  bool odd_late = false;
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    if (r * kSortThreads >= n) break;
    const int round = r & 1;
    const int i = r * kSortThreads + tid;
    bool keep = false, outside = false;
    float key = 0.f;
    const typename Source::Rec& P = P_buf[r & 1];
    const int p = my_id[r];
    if (r + 1 < kRounds && i + kSortThreads < n)
      P_buf[(r + 1) & 1] = src.load(((unsigned)my_id[r + 1] < (unsigned)num_prims) ? my_id[r + 1] : 0);
    const bool known = (unsigned)p < (unsigned)num_prims;
    if constexpr (PYR) py = pyramid_from_word(pyramid_word);
    if (i < n) {
      outside = faces && known && outside_pyramid(py, P, cull_r2);
      keep = !outside;
      if (keep) key = !known ? kInvalidKey : src.key(family, dx, dy, dz, P);
    }
    const uint32_t kb = float_to_bits(key);
    const bool late = keep && kb >= invalid_bits;
    const bool front = keep && !late;
    // (the builtin on the predicates themselves: __ballot() takes an int, and the predicate's way through a
    // register and back is two vector instructions per vote)
    const unsigned long long mf = __builtin_amdgcn_ballot_w64(front), ml = __builtin_amdgcn_ballot_w64(late);
    if (lane == 0) s_wave_cnt[round][wave] = __popcll(mf) | (__popcll(ml) << 16);
    __syncthreads();                                     // (the two count buffers alternate: one barrier per round)
    int before = survivors, total = 0;
#pragma unroll
    for (int v = 0; v < kSortThreads / 64; ++v) {
      const int c = __builtin_amdgcn_readfirstlane(s_wave_cnt[round][v]);     // (the same word in every lane)
      before += (v < wave) ? c : 0;
      total += c;
    }
    const unsigned long long below = (1ull << lane) - 1ull;
    const int f_before = (before & 0xffff) + __popcll(mf & below);
    const int l_before = (before >> 16) + __popcll(ml & below);
    const unsigned long long entry = ((unsigned long long)kb << 32) | (unsigned)(ASC ? p : i);
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
    survivors += total;
  }
  int nv = survivors & 0xffff, nl = survivors >> 16;
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

  // ---- order of the ordinary survivors.  Usual case: a counting pass into 512 buckets that are linear in the
  //      key bits between the smallest and the largest key (monotone, so bucket order is key order), then every
  //      entry ranks itself among the entries of its own bucket by its (key, list position) word.  The work of
  //      that last step is the sum of the squared bucket sizes; when keys pile up in few buckets (or a late key
  //      is not the invalid key, which the late stream's list order would misplace) the bitonic network below
  //      sorts instead.
  // (two buckets per thread: their counts, offsets and cursors are 16-bit halves of one word -- a list holds at
  // most kSortMax <= 65,535 entries, so a half never carries into its neighbour)
  constexpr int kBuckets = 2 * kSortThreads;
  const uint32_t kmin = s_kmin;
  const float bucket_scale = (float)kBuckets / ((float)(s_kmax - kmin) + 1.f);
  auto bucket_of = [&](unsigned long long w) {
    const int b = (int)((float)((uint32_t)(w >> 32) - kmin) * bucket_scale);
    return b < kBuckets - 1 ? b : kBuckets - 1;
  };
  auto half_of = [](int word, int b) { return (word >> ((b & 1) << 4)) & 0xffff; };
  auto one_in = [](int b) { return 1 << ((b & 1) << 4); };
  bool network = (s_flags & 1) != 0;
  const bool ranked = !network && nv > 1;
  if (ranked) {
    s_cnt[tid] = 0;
    __syncthreads();
    for (int i = tid; i < nv; i += kSortThreads) {
      const int b = bucket_of(s_key[i]);
      atomicAdd(&s_cnt[b >> 1], one_in(b));
    }
    __syncthreads();
    const int c0 = s_cnt[tid] & 0xffff, c1 = (s_cnt[tid] >> 16) & 0xffff;
    const int c = c0 + c1;
    int incl = c, pairs = c0 * c0 + c1 * c1;
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
    s_off[tid] = excl | ((excl + c0) << 16);
    s_cnt[tid] = excl | ((excl + c0) << 16);             // from here on: the buckets' fill cursors
    network = s_pairs > kRankPairsMax;
    __syncthreads();
    if (!network) {
      for (int i = tid; i < nv; i += kSortThreads) {
        const int b = bucket_of(s_key[i]);
        s_perm[half_of(atomicAdd(&s_cnt[b >> 1], one_in(b)), b)] = (uint16_t)i;
      }
      __syncthreads();
      for (int a = tid; a < nv; a += kSortThreads) {
        const int ia = s_perm[a];
        const unsigned long long wa = s_key[ia];
        const int b = bucket_of(wa);
        const int lo = half_of(s_off[b >> 1], b), hi = half_of(s_cnt[b >> 1], b);   // the cursor ended at the bucket's end
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
      sorted_ids[start + i] = ASC ? (int)(w & 0xffffffffu) : cand[start + (int)(w & 0xffffffffu)];
      if (sorted_keys) sorted_keys[start + i] = bits_to_float((uint32_t)(w >> 32));
    } else if (i >= n) {
      sorted_ids[start + i] = cand[start + i];     // beyond the sort capacity: list order, never culled
      if (sorted_keys) sorted_keys[start + i] = kInvalidKey;
    }
  }
}

template <int kSortMax, bool PYR, bool ASC = false>
__device__ __forceinline__ void sort_one_tile(SortLds<kSortMax>& lds,
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const SortRec* __restrict__ frame, const TilePyramidRec* __restrict__ pyramids, const int32_t* __restrict__ cand,
    const int32_t* __restrict__ offsets, const int32_t* __restrict__ ends, const TileGeom& g, int family, int capacity,
    float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids, float* __restrict__ sorted_keys, int tile) {
  const int start = offsets[tile];
  const int len = ends[tile] - start;
  if (len <= 0) return;
  const int n = len < capacity ? len : capacity;
  const int pc = centre_pixel(g, tile);
  const float ox = rays_o[pc * 3 + 0], oy = rays_o[pc * 3 + 1], oz = rays_o[pc * 3 + 2];
  const float dx = rays_d[pc * 3 + 0], dy = rays_d[pc * 3 + 1], dz = rays_d[pc * 3 + 2];
  if (frame_records_hold(frame, ox, oy, oz))
    sort_one_tile_from<kSortMax, PYR, ASC>(lds, FromFrameRecord{frame + 1}, rays_o, rays_d, pyramids, g, tile, dx, dy, dz, cand,
                                 family, cull_r2, num_prims, sorted_ids, sorted_keys, start, len, n);
  else
    sort_one_tile_from<kSortMax, PYR, ASC>(lds, FromPrimRecord{prims, ox, oy, oz}, rays_o, rays_d, pyramids, g, tile, dx, dy, dz,
                                 cand, family, cull_r2, num_prims, sorted_ids, sorted_keys, start, len, n);
}

}  // namespace mlpsp
