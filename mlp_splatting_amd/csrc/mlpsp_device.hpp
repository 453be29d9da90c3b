// Device-side arithmetic shared by the gfx950 kernels of the tile renderer.
//
// Everything here is plain IEEE f32: add, mul, fma, divide (correctly rounded), compare, select
// and integer bit operations.  No native transcendental instruction is used, so a host program
// that performs the same sequence of operations obtains the same bits.  All translation units
// that include this header must be compiled with -ffp-contract=off: a multiply followed by an
// add is two roundings unless fmaf() is written.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlpsp {

constexpr float kTransmittanceFloor = 1e-3f;  // pixel stops once T < 1e-3 (np_tile_kernels.cu:2026)
constexpr float kInvalidKey = 1e30f;          // sort key of primitives behind the ray (np_tile_kernels.cu:514-517)

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t float_to_bits(float x) { return __float_as_uint(x); }

// e^x: x < -87 -> 0, x > 88 -> +inf, NaN -> NaN.  k = rint(x log2 e), r = x - k ln2 in two
// parts, degree-7 Taylor polynomial, scaling by 2^k through the exponent field.
__device__ __forceinline__ float det_exp(float x) {
  const float xc = fminf(fmaxf(x, -87.0f), 88.0f);
  const float kf = __builtin_rintf(xc * 1.44269504f);
  float r = fmaf(kf, -0.693145752f, xc);
  r = fmaf(kf, -1.42860677e-06f, r);
  float p = 1.98412698e-04f;
  p = fmaf(p, r, 1.38888889e-03f);
  p = fmaf(p, r, 8.33333333e-03f);
  p = fmaf(p, r, 4.16666667e-02f);
  p = fmaf(p, r, 1.66666667e-01f);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  const int k = (int)kf;
  float y = p * bits_to_float((uint32_t)(k + 127) << 23);
  y = (x < -87.0f) ? 0.0f : y;
  y = (x > 88.0f) ? __builtin_inff() : y;
  return (x != x) ? x : y;
}

// sin and cos of x in radians; |x| > 65536 or non-finite -> NaN.  Cody-Waite reduction by
// multiples of pi/2 in three parts, Taylor polynomials on [-pi/4, pi/4], quadrant fix-up.
__device__ __forceinline__ void det_sincos(float x, float& s_out, float& c_out) {
  const float kf = __builtin_rintf(x * 0.636619772f);
  float r = fmaf(kf, -1.5703125f, x);
  r = fmaf(kf, -4.83751297e-04f, r);
  r = fmaf(kf, -7.54978995e-08f, r);
  const float z = r * r;
  float ps = 2.75573192e-06f;
  ps = fmaf(ps, z, -1.98412698e-04f);
  ps = fmaf(ps, z, 8.33333333e-03f);
  ps = fmaf(ps, z, -1.66666667e-01f);
  const float s = fmaf(r * z, ps, r);
  float pc = -2.75573192e-07f;
  pc = fmaf(pc, z, 2.48015873e-05f);
  pc = fmaf(pc, z, -1.38888889e-03f);
  pc = fmaf(pc, z, 4.16666667e-02f);
  const float c = fmaf(z * z, pc, fmaf(z, -0.5f, 1.0f));
  const int q = ((int)kf) & 3;
  const float sv = (q & 1) ? c : s;
  const float cv = (q & 1) ? s : c;
  const float so = (q & 2) ? -sv : sv;
  const float co = ((q + 1) & 2) ? -cv : cv;
  const bool ok = __builtin_fabsf(x) <= 65536.0f;
  s_out = ok ? so : __builtin_nanf("");
  c_out = ok ? co : __builtin_nanf("");
}

// log(u), u normal positive finite: u = m 2^e with m in (sqrt(1/2), sqrt(2)], log m = 2 atanh(s).
__device__ __forceinline__ float det_log_pos(float u) {
  const uint32_t b = float_to_bits(u);
  int e = (int)(b >> 23) - 127;
  float m = bits_to_float((b & 0x007fffffu) | 0x3f800000u);
  const bool big = m > 1.41421354f;
  m = big ? m * 0.5f : m;
  e = big ? e + 1 : e;
  const float f = m - 1.0f;
  const float s = f / (2.0f + f);
  const float z = s * s;
  float p = 0.111111111f;
  p = fmaf(p, z, 0.142857143f);
  p = fmaf(p, z, 0.2f);
  p = fmaf(p, z, 0.333333333f);
  const float two_s = s + s;
  const float lm = fmaf(two_s * z, p, two_s);
  const float ef = (float)e;
  return fmaf(ef, 0.693145752f, fmaf(ef, 1.42860677e-06f, lm));
}

// log(1 + x), x >= 0.
__device__ __forceinline__ float det_log1p_pos(float x) {
  const float u = 1.0f + x;
  const float v = det_log_pos(u) + (x - (u - 1.0f)) / u;
  return (u == 1.0f) ? x : v;
}

// np_tile_kernels.cu:75-77
__device__ __forceinline__ float sigmoid(float x) { return 1.0f / (1.0f + det_exp(-x)); }

// np_tile_kernels.cu:79-83
__device__ __forceinline__ float softplus(float x) {
  const float e = det_exp(x);
  const float mid = det_log1p_pos(e);
  float y = (x < -20.f) ? e : mid;
  y = (x > 20.f) ? x : y;
  return y;
}

struct Vec3 {
  float x, y, z;
};

// v + w t + q x t with t = 2 q x v (np_tile_kernels.cu:416-428); every product and sum rounds.
__device__ __forceinline__ Vec3 quat_rotate(float qw, float qx, float qy, float qz, Vec3 v) {
  const float tx = 2.f * (qy * v.z - qz * v.y);
  const float ty = 2.f * (qz * v.x - qx * v.z);
  const float tz = 2.f * (qx * v.y - qy * v.x);
  Vec3 r;
  r.x = (v.x + qw * tx) + (qy * tz - qz * ty);
  r.y = (v.y + qw * ty) + (qz * tx - qx * tz);
  r.z = (v.z + qw * tz) + (qx * ty - qy * tx);
  return r;
}
__device__ __forceinline__ Vec3 quat_rotate_conj(float qw, float qx, float qy, float qz, Vec3 v) {
  return quat_rotate(qw, -qx, -qy, -qz, v);
}

// One primitive's geometry as the kernels consume it: 128 bytes, written by the prepare kernel.
// First 64 bytes, for the exactly rounded paths and the sort: m = exp(-2 log_s) is the diagonal of the precision
// matrix, s2 = exp(2 log_s) the squared semi-axes (used only by the conservative tile culling of the sort kernel).
// Second 64 bytes (one cache line, one scalar load), for the reduced-precision render path only: the centre again
// and rs[k] = exp(-log_s[k]) * row k of R(q)^T, the world -> local rotation with the inverse scales folded in, so
// that |rs (x - c)|^2 is the Mahalanobis distance (three dot products per vector instead of the quaternion form,
// which the exact paths must keep to reproduce the reference's roundings).
struct __attribute__((aligned(128))) PrimRecord {
  float cx, cy, cz, mx;
  float my, mz, qw, qx;
  float qy, qz, lgx, lgy;
  float lgz, s2x, s2y, s2z;
  float fcx, fcy, fcz;
  float rs[3][3];
  float pad[4];
};
static_assert(sizeof(PrimRecord) == 128, "record size is part of the C ABI");

struct HitInfo {
  float t, dx, dy, dz, qlx, qly, qlz, decay;
};

// Ray against rotated ellipsoid (np_tile_kernels.cu:659-711).  Returns decay > thr.
__device__ __forceinline__ bool hit_rot(float rox, float roy, float roz, float rdx, float rdy, float rdz,
                                        const PrimRecord& P, float thr, HitInfo& h) {
  const Vec3 v = {P.cx - rox, P.cy - roy, P.cz - roz};
  const Vec3 vl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, v);
  const Vec3 dl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, Vec3{rdx, rdy, rdz});
  const float denom = fmaf(dl.x * dl.x, P.mx, fmaf(dl.y * dl.y, P.my, (dl.z * dl.z) * P.mz));
  const float numer = fmaf(dl.x * vl.x, P.mx, fmaf(dl.y * vl.y, P.my, (dl.z * vl.z) * P.mz));
  const float t = numer / denom;
  const float px = rox + t * rdx;
  const float py = roy + t * rdy;
  const float pz = roz + t * rdz;
  h.t = t;
  h.dx = P.cx - px;
  h.dy = P.cy - py;
  h.dz = P.cz - pz;
  const Vec3 ql = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, Vec3{h.dx, h.dy, h.dz});
  h.qlx = ql.x;
  h.qly = ql.y;
  h.qlz = ql.z;
  const float r2 = fmaxf(((ql.x * ql.x) * P.mx + (ql.y * ql.y) * P.my) + (ql.z * ql.z) * P.mz, 0.f);
  h.decay = det_exp(-0.5f * r2);
  return !(denom <= 1e-20f) && !(t <= 0.f) && (h.decay > thr);
}

// Mahalanobis t* of the tile-centre ray (np_tile_kernels.cu:483-518, then :1973).
__device__ __forceinline__ float key_tstar(float ox, float oy, float oz, float dx, float dy, float dz,
                                           const PrimRecord& P) {
  const Vec3 v = {P.cx - ox, P.cy - oy, P.cz - oz};
  const Vec3 vl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, v);
  const Vec3 dl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, Vec3{dx, dy, dz});
  const float denom = fmaf(dl.x * dl.x, P.mx, fmaf(dl.y * dl.y, P.my, (dl.z * dl.z) * P.mz));
  const float numer = fmaf(dl.x * vl.x, P.mx, fmaf(dl.y * vl.y, P.my, (dl.z * vl.z) * P.mz));
  const float t = numer / denom;
  return (denom > 1e-20f && t > 0.f) ? t : kInvalidKey;
}

// Plain centre-ray depth (np_tile_kernels.cu:5538-5542).
__device__ __forceinline__ float key_depth(float ox, float oy, float oz, float dx, float dy, float dz,
                                           const PrimRecord& P) {
  const float vx = P.cx - ox, vy = P.cy - oy, vz = P.cz - oz;
  const float k = fmaf(vx, dx, fmaf(vy, dy, vz * dz));
  return (k > 0.f) ? k : kInvalidKey;
}

// Tetrahedral softmax gates on the local hit coordinate (np_tile_kernels.cu:97-124).
__device__ __forceinline__ void tetra_gates(float qlx, float qly, float qlz, float lgx, float lgy, float lgz,
                                            float beta, float temp, float g[4]) {
  const float ux = fminf(1.f, fmaxf(-1.f, qlx / (beta * det_exp(lgx) + 1e-6f)));
  const float uy = fminf(1.f, fmaxf(-1.f, qly / (beta * det_exp(lgy) + 1e-6f)));
  const float uz = fminf(1.f, fmaxf(-1.f, qlz / (beta * det_exp(lgz) + 1e-6f)));
  const float l0 = temp * ((ux + uy) + uz);
  const float l1 = temp * ((ux - uy) - uz);
  const float l2 = temp * ((-ux + uy) - uz);
  const float l3 = temp * ((-ux - uy) + uz);
  const float lm = fmaxf(fmaxf(l0, l1), fmaxf(l2, l3));
  const float e0 = det_exp(l0 - lm), e1 = det_exp(l1 - lm), e2 = det_exp(l2 - lm), e3 = det_exp(l3 - lm);
  const float inv = 1.f / fmaxf(((e0 + e1) + e2) + e3, 1e-8f);
  g[0] = e0 * inv;
  g[1] = e1 * inv;
  g[2] = e2 * inv;
  g[3] = e3 * inv;
}

// Per-pixel compositing state and one blend step (np_tile_kernels.cu:2092-2103, 5669-5671).
struct PixelAcc {
  float cr, cg, cb, trans, w_acc, t_acc;
};

__device__ __forceinline__ float blend_step(PixelAcc& a, float o0, float o1, float o2, float o3, float decay,
                                            float t) {
  const float sigma = softplus(o3) * decay;
  const float alpha = 1.f - det_exp(-sigma);
  const float w = a.trans * alpha;
  a.w_acc = fmaf(1.f, w, a.w_acc);
  a.t_acc = fmaf(w, t, a.t_acc);
  a.cr = fmaf(w, sigmoid(o0), a.cr);
  a.cg = fmaf(w, sigmoid(o1), a.cg);
  a.cb = fmaf(w, sigmoid(o2), a.cb);
  a.trans = a.trans * (1.f - alpha);
  return w;
}

// Tile <-> pixel mapping shared by every kernel (np_tile_kernels.cu:1862-1873, 1883-1886).
struct TileGeom {
  int W, H, TW, TH, ntx, nty;
};

// Element `i` of a [*, 3] float array as ONE 12-byte access: the rays (or pixels) of a tile lie 12 bytes apart over
// several image rows, and what such reads cost is the number of load instructions (the sort's check of a tile's 64
// rays, three 4-byte loads per array and lane, measured 11 us per frame more than this form).
struct __attribute__((packed, aligned(4))) Float3 {
  float x, y, z;
};
__device__ __forceinline__ Float3 load3(const float* __restrict__ base, long long i) {
  return *reinterpret_cast<const Float3*>(base + i * 3);
}
__device__ __forceinline__ void store3(float* __restrict__ base, long long i, float x, float y, float z) {
  Float3 v;
  v.x = x;
  v.y = y;
  v.z = z;
  *reinterpret_cast<Float3*>(base + i * 3) = v;
}

// torch.nn.functional.normalize(d, dim=-1) of one direction, bit for bit (scannet/cumodel.py:1088): the squares are
// summed as (x^2 + z^2) + y^2 -- the order of torch's reduction over a last dimension of three -- then an exactly
// rounded square root and three exactly rounded divisions.
__device__ __forceinline__ void unit_direction(float x, float y, float z, float& ux, float& uy, float& uz) {
  const float den = fmaxf(sqrtf((x * x + z * z) + y * y), 1e-12f);
  ux = x / den;
  uy = y / den;
  uz = z / den;
}
__device__ __forceinline__ int centre_pixel(const TileGeom& g, int tile) {
  const int tx = tile % g.ntx, ty = tile / g.ntx;
  const int cx = min(tx * g.TW + (g.TW >> 1), g.W - 1);
  const int cy = min(ty * g.TH + (g.TH >> 1), g.H - 1);
  return cy * g.W + cx;
}

}  // namespace mlpsp
