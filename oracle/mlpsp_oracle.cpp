// CPU oracle for the MLP-Splatting tile-based forward renderer.
//
// TEST INFRASTRUCTURE ONLY.  This file restates, on the CPU, the algorithm of the reference
// renderer so that the HIP kernels can be checked against it.  Nothing in the shipped package
// may include, link or call it; only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
// bench.py do.
//
// Every function cites the reference text it follows (paths relative to the reference
// repository root).  The reference leaves three things open, and this file fixes them:
//   * `a*b+c` expressions outside explicit fmaf() are contracted or not at nvcc's discretion;
//     here every operation is written out (fmaf where the reference writes fmaf, separate
//     multiply and add otherwise) and the file is compiled with -ffp-contract=off.
//   * __expf/__sinf/__cosf/log1pf are NVIDIA intrinsics with no bit-level specification;
//     here they are replaced by det_exp/det_sincos/det_log1p below, built from IEEE
//     add/mul/fma/div only, so that a GPU implementation of the same recipe is bit-identical.
//   * torch's matmul in the culling code has no specified accumulation order; here the
//     4-term dot products are explicit fma chains.
//
// Parity status per function (what pins it is in tests/test_oracle_*.py):
//   det_exp, det_sincos, det_log1p, sigmoid, softplus ... pinned against libm (double) to <= 2 ulp
//   quat rotation, hit test, sort keys ................... pinned by closed forms + rotation invariance
//   MLP .................................................. pinned against an einsum restatement
//   compositing / early termination ...................... pinned by geometric-series closed forms
//   ordering / capacity / validation ..................... pinned by the reference tests' cases
//   legacy + tile-view binning ........................... pinned by brute force over the dense predicate
//   ray-cone binning ..................................... pinned by the reference's own brute-force test
//   gates / feature ...................................... pinned by softmax closed form + framebuffer sum
//   training records ..................................... pinned by recomposition (sum T a c = rgb,
//       T' = T (1 - a)), the forward image within 2e-6, masks against an einsum restatement
//   reverse compositing over records ..................... pinned against float64 autograd through a
//       differentiable restatement of the compositing (tests/test_oracle_render.py)
//   pruning statistics ................................... pinned by the geometric-series weights of
//       stacked identical primitives and by sum_p sum_w[p] = sum_pixels alpha
//   bf16/fp16 mixed-precision MLP ........................ pinned against a numpy emulation of the
//       rounding points; the reference entry point itself (render_tiles_rgb_wmma) has no test in
//       the reference: "parity unpinned" beyond the stated tolerances.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <immintrin.h>
#include <omp.h>

#define ORACLE_API extern "C" __attribute__((visibility("default")))

namespace {

inline uint32_t f2u(float x) { uint32_t u; std::memcpy(&u, &x, 4); return u; }
inline float u2f(uint32_t u) { float x; std::memcpy(&x, &u, 4); return x; }

// ------------------------------------------------------------------------------------------
// Deterministic elementary functions (stand-ins for __expf, __sinf, __cosf, log1pf used at
// scannet/cuda/np_tile_kernels.cu:75-83, 676-678, 709, 2059-2060, 2094).
// ------------------------------------------------------------------------------------------

// e^x.  x < -87 -> 0, x > 88 -> +inf, NaN -> NaN.  k = rint(x*log2e); r = x - k*ln2 (two-part);
// degree-7 Taylor polynomial in Horner form; scale by 2^k built from the exponent bits.
inline float det_exp(float x) {
  if (x != x) return x;
  if (x < -87.0f) return 0.0f;
  if (x > 88.0f) return INFINITY;
  const float kf = rintf(x * 1.44269504f);
  float r = fmaf(kf, -0.693145752f, x);
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
  return p * u2f((uint32_t)(k + 127) << 23);
}

// sin and cos of x (radians).  |x| > 65536 or non-finite -> NaN for both.
// k = rint(x*2/pi); three-part Cody-Waite reduction; Taylor polynomials on [-pi/4, pi/4].
inline void det_sincos(float x, float* s_out, float* c_out) {
  if (!(fabsf(x) <= 65536.0f)) { *s_out = NAN; *c_out = NAN; return; }
  const float kf = rintf(x * 0.636619772f);
  float r = fmaf(kf, -1.5703125f, x);
  r = fmaf(kf, -4.83751297e-04f, r);
  r = fmaf(kf, -7.54978995e-08f, r);
  const float z = r * r;
  float ps = 2.75573192e-06f;            // 1/9!
  ps = fmaf(ps, z, -1.98412698e-04f);    // -1/7!
  ps = fmaf(ps, z, 8.33333333e-03f);     // 1/5!
  ps = fmaf(ps, z, -1.66666667e-01f);    // -1/3!
  const float s = fmaf(r * z, ps, r);
  float pc = -2.75573192e-07f;           // -1/10!
  pc = fmaf(pc, z, 2.48015873e-05f);     // 1/8!
  pc = fmaf(pc, z, -1.38888889e-03f);    // -1/6!
  pc = fmaf(pc, z, 4.16666667e-02f);     // 1/4!
  const float c = fmaf(z * z, pc, fmaf(z, -0.5f, 1.0f));
  const int q = ((int)kf) & 3;
  const float sv = (q & 1) ? c : s;
  const float cv = (q & 1) ? s : c;
  *s_out = (q & 2) ? -sv : sv;
  *c_out = ((q + 1) & 2) ? -cv : cv;
}

// log(u) for normal positive finite u: u = m*2^e, m in (sqrt(.5), sqrt(2)];
// log m = 2 atanh(s), s = (m-1)/(m+1), series to s^9.
inline float det_log_pos(float u) {
  const uint32_t b = f2u(u);
  int e = (int)(b >> 23) - 127;
  float m = u2f((b & 0x007fffffu) | 0x3f800000u);
  if (m > 1.41421354f) { m = m * 0.5f; e += 1; }
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

// log(1+x) for x >= 0 (finite): log(u) + (x-(u-1))/u with u = fl(1+x).
inline float det_log1p_pos(float x) {
  const float u = 1.0f + x;
  if (u == 1.0f) return x;
  return det_log_pos(u) + (x - (u - 1.0f)) / u;
}

// scannet/cuda/np_tile_kernels.cu:75-77
inline float o_sigmoid(float x) { return 1.0f / (1.0f + det_exp(-x)); }

// scannet/cuda/np_tile_kernels.cu:79-83
inline float o_softplus(float x) {
  if (x > 20.f) return x;
  if (x < -20.f) return det_exp(x);
  return det_log1p_pos(det_exp(x));
}

// ------------------------------------------------------------------------------------------
// Geometry
// ------------------------------------------------------------------------------------------
struct V3 { float x, y, z; };

// scannet/cuda/np_tile_kernels.cu:416-428.  Every product and sum is a separate rounding.
inline V3 quat_rotate(float qw, float qx, float qy, float qz, V3 v) {
  const float tx = 2.f * (qy * v.z - qz * v.y);
  const float ty = 2.f * (qz * v.x - qx * v.z);
  const float tz = 2.f * (qx * v.y - qy * v.x);
  V3 r;
  r.x = (v.x + qw * tx) + (qy * tz - qz * ty);
  r.y = (v.y + qw * ty) + (qz * tx - qx * tz);
  r.z = (v.z + qw * tz) + (qx * ty - qy * tx);
  return r;
}
// scannet/cuda/np_tile_kernels.cu:430-435
inline V3 quat_rotate_conj(float qw, float qx, float qy, float qz, V3 v) {
  return quat_rotate(qw, -qx, -qy, -qz, v);
}

struct Prim {
  float cx, cy, cz;
  float lgx, lgy, lgz;
  float qw, qx, qy, qz;
  float mx, my, mz;  // exp(-2*log_s), np_tile_kernels.cu:676-678
};

inline Prim load_prim(const float* pos, const float* logs, const float* quats, int p) {
  Prim P;
  P.cx = pos[p * 3 + 0]; P.cy = pos[p * 3 + 1]; P.cz = pos[p * 3 + 2];
  P.lgx = logs[p * 3 + 0]; P.lgy = logs[p * 3 + 1]; P.lgz = logs[p * 3 + 2];
  P.qw = quats[p * 4 + 0]; P.qx = quats[p * 4 + 1]; P.qy = quats[p * 4 + 2]; P.qz = quats[p * 4 + 3];
  P.mx = det_exp(-2.f * P.lgx); P.my = det_exp(-2.f * P.lgy); P.mz = det_exp(-2.f * P.lgz);
  return P;
}

struct Hit { float t, dx, dy, dz, qlx, qly, qlz, decay; };

// scannet/cuda/np_tile_kernels.cu:659-711 (hit_and_features_rot)
inline bool hit_rot(float rox, float roy, float roz, float rdx, float rdy, float rdz,
                    const Prim& P, float thr, Hit& h) {
  const V3 v = {P.cx - rox, P.cy - roy, P.cz - roz};
  const V3 vl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, v);
  const V3 dl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, V3{rdx, rdy, rdz});
  const float denom = fmaf(dl.x * dl.x, P.mx, fmaf(dl.y * dl.y, P.my, (dl.z * dl.z) * P.mz));
  if (denom <= 1e-20f) return false;
  const float numer = fmaf(dl.x * vl.x, P.mx, fmaf(dl.y * vl.y, P.my, (dl.z * vl.z) * P.mz));
  const float t = numer / denom;
  if (t <= 0.f) return false;
  const float px = rox + t * rdx;
  const float py = roy + t * rdy;
  const float pz = roz + t * rdz;
  h.t = t;
  h.dx = P.cx - px; h.dy = P.cy - py; h.dz = P.cz - pz;
  const V3 ql = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, V3{h.dx, h.dy, h.dz});
  h.qlx = ql.x; h.qly = ql.y; h.qlz = ql.z;
  const float r2 = fmaxf(((ql.x * ql.x) * P.mx + (ql.y * ql.y) * P.my) + (ql.z * ql.z) * P.mz, 0.f);
  h.decay = det_exp(-0.5f * r2);
  return h.decay > thr;
}

// scannet/cuda/np_tile_kernels.cu:483-518 (tstar_key_tilecenter) followed by :1973
inline float key_tstar(float ox, float oy, float oz, float dx, float dy, float dz, const Prim& P) {
  const V3 v = {P.cx - ox, P.cy - oy, P.cz - oz};
  const V3 vl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, v);
  const V3 dl = quat_rotate_conj(P.qw, P.qx, P.qy, P.qz, V3{dx, dy, dz});
  const float denom = fmaf(dl.x * dl.x, P.mx, fmaf(dl.y * dl.y, P.my, (dl.z * dl.z) * P.mz));
  const float numer = fmaf(dl.x * vl.x, P.mx, fmaf(dl.y * vl.y, P.my, (dl.z * vl.z) * P.mz));
  if (denom <= 1e-20f) return 1e30f;
  const float t = numer / denom;
  return (t > 0.f) ? t : 1e30f;
}

// scannet/cuda/np_tile_kernels.cu:5538-5542 (plain centre-ray depth key)
inline float key_depth(float ox, float oy, float oz, float dx, float dy, float dz, const Prim& P) {
  const float vx = P.cx - ox, vy = P.cy - oy, vz = P.cz - oz;
  const float k = fmaf(vx, dx, fmaf(vy, dy, vz * dz));
  return (k > 0.f) ? k : 1e30f;
}

// scannet/cuda/np_tile_kernels.cu:97-124 (semantic_tetra_gates)
inline void tetra_gates(float qlx, float qly, float qlz, float lgx, float lgy, float lgz,
                        float beta, float temp, float g[4]) {
  auto clamp = [](float x) { return fminf(1.f, fmaxf(-1.f, x)); };
  const float ux = clamp(qlx / (beta * det_exp(lgx) + 1e-6f));
  const float uy = clamp(qly / (beta * det_exp(lgy) + 1e-6f));
  const float uz = clamp(qlz / (beta * det_exp(lgz) + 1e-6f));
  const float l0 = temp * ((ux + uy) + uz);
  const float l1 = temp * ((ux - uy) - uz);
  const float l2 = temp * ((-ux + uy) - uz);
  const float l3 = temp * ((-ux - uy) + uz);
  const float lm = fmaxf(fmaxf(l0, l1), fmaxf(l2, l3));
  const float e0 = det_exp(l0 - lm), e1 = det_exp(l1 - lm), e2 = det_exp(l2 - lm), e3 = det_exp(l3 - lm);
  const float inv = 1.f / fmaxf(((e0 + e1) + e2) + e3, 1e-8f);
  g[0] = e0 * inv; g[1] = e1 * inv; g[2] = e2 * inv; g[3] = e3 * inv;
}

// ------------------------------------------------------------------------------------------
// MLP
// ------------------------------------------------------------------------------------------
constexpr int MAXH = 64;  // np_tile_kernels.cu:5922 (Hcap <= 64 in the feature/depth kernels)

// round-to-nearest-even f32 -> bf16 -> f32 (__float2bfloat16_rn, rgb_wmma.cuh:17-19)
inline float round_bf16(float x) {
  uint32_t u = f2u(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return u2f(u | 0x00400000u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return u2f(u & 0xffff0000u);
}
// round-to-nearest-even f32 -> fp16 -> f32 (__float2half_rn, rgb_wmma.cuh:14-16)
inline float round_f16(float x) {
  return _cvtsh_ss(_cvtss_sh(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
}
inline float round_op(float x, int precision) {
  return precision == 1 ? round_bf16(x) : (precision == 2 ? round_f16(x) : x);
}

struct MlpView {
  const float *W1, *b1, *W2, *b2, *W3, *b3;  // already offset to the primitive
  int H, IN, F;
};

// Scalar f32 MLP, operation order of scannet/cuda/np_tile_kernels.cu:2047-2089.
inline void mlp_f32(const float x6[6], const float* freq, const float* att, const MlpView& M, float out[4]) {
  float h1[MAXH], h2[MAXH];
  const int H = M.H, IN = M.IN, F = M.F, cos_off = IN / 2;
  for (int h = 0; h < H; ++h) h1[h] = M.b1[h];
  for (int c = 0; c < 6; ++c) {
    for (int f = 0; f < F; ++f) {
      const float xproj = (x6[c] * freq[f]) * att[f];
      const int j = c * F + f;
      float s, co;
      det_sincos(xproj, &s, &co);
      for (int h = 0; h < H; ++h) {
        const float* Wi = M.W1 + (size_t)h * IN;
        h1[h] = fmaf(Wi[j], s, h1[h]);
        h1[h] = fmaf(Wi[j + cos_off], co, h1[h]);
      }
    }
  }
  for (int h = 0; h < H; ++h) h1[h] = h1[h] > 0.f ? h1[h] : 0.f;
  for (int o = 0; o < H; ++o) {
    float acc = M.b2[o];
    const float* row = M.W2 + (size_t)o * H;
    for (int h = 0; h < H; ++h) acc = fmaf(row[h], h1[h], acc);
    h2[o] = acc > 0.f ? acc : 0.f;
  }
  float o0 = M.b3[0], o1 = M.b3[1], o2 = M.b3[2], o3 = M.b3[3];
  for (int h = 0; h < H; ++h) {
    const float hi = h2[h];
    o0 = fmaf(M.W3[0 * H + h], hi, o0);
    o1 = fmaf(M.W3[1 * H + h], hi, o1);
    o2 = fmaf(M.W3[2 * H + h], hi, o2);
    o3 = fmaf(M.W3[3 * H + h], hi, o3);
  }
  out[0] = o0; out[1] = o1; out[2] = o2; out[3] = o3;
}

// The MLP as the record kernels evaluate it (mlp_eval_rgb_sigma, scannet/cuda/np_tile_kernels.cu:313-381):
// layer 1 and 3 as above, layer 2 as bias + (fma chain started at zero) (:349-353, row_dot_vec :208-212),
// which rounds differently from the forward kernels' chain started at the bias; masks[l] has bit h set
// iff hidden unit h of layer l+1 is positive after ReLU (:371-379).
inline void mlp_f32_records(const float x6[6], const float* freq, const float* att, const MlpView& M, float out[4],
                            uint32_t masks[2]) {
  float h1[MAXH], h2[MAXH];
  const int H = M.H, IN = M.IN, F = M.F, cos_off = IN / 2;
  for (int h = 0; h < H; ++h) h1[h] = M.b1[h];
  for (int c = 0; c < 6; ++c) {
    for (int f = 0; f < F; ++f) {
      const float xproj = (x6[c] * freq[f]) * att[f];
      const int j = c * F + f;
      float s, co;
      det_sincos(xproj, &s, &co);
      for (int h = 0; h < H; ++h) {
        const float* Wi = M.W1 + (size_t)h * IN;
        h1[h] = fmaf(Wi[j], s, h1[h]);
        h1[h] = fmaf(Wi[j + cos_off], co, h1[h]);
      }
    }
  }
  for (int h = 0; h < H; ++h) h1[h] = h1[h] > 0.f ? h1[h] : 0.f;
  for (int o = 0; o < H; ++o) {
    const float* row = M.W2 + (size_t)o * H;
    float dot = 0.f;
    for (int h = 0; h < H; ++h) dot = fmaf(row[h], h1[h], dot);
    const float acc = M.b2[o] + dot;
    h2[o] = acc > 0.f ? acc : 0.f;
  }
  float o0 = M.b3[0], o1 = M.b3[1], o2 = M.b3[2], o3 = M.b3[3];
  for (int h = 0; h < H; ++h) {
    const float hi = h2[h];
    o0 = fmaf(M.W3[0 * H + h], hi, o0);
    o1 = fmaf(M.W3[1 * H + h], hi, o1);
    o2 = fmaf(M.W3[2 * H + h], hi, o2);
    o3 = fmaf(M.W3[3 * H + h], hi, o3);
  }
  out[0] = o0; out[1] = o1; out[2] = o2; out[3] = o3;
  uint32_t m1 = 0, m2 = 0;
  for (int h = 0; h < H && h < 32; ++h) {
    if (h1[h] > 0.f) m1 |= (1u << h);
    if (h2[h] > 0.f) m2 |= (1u << h);
  }
  masks[0] = m1; masks[1] = m2;
}

// Mixed-precision MLP, rounding points of scannet/cuda/rgb_wmma.cuh:144-213: encoded inputs and
// all weights rounded to the operand type; products accumulated in f32 (from zero, k ascending;
// the reference's MMA order is unspecified); bias added in f32; ReLU; hidden activations rounded
// to the operand type again; layer-3 result + b3 stays f32.
inline void mlp_mixed(const float x6[6], const float* freq, const float* att, const MlpView& M,
                      int precision, float out[4]) {
  float enc[12 * 16];
  float h1[MAXH], h2[MAXH];
  const int H = M.H, IN = M.IN, F = M.F, cos_off = IN / 2;
  for (int c = 0; c < 6; ++c)
    for (int f = 0; f < F; ++f) {
      float s, co;
      det_sincos((x6[c] * freq[f]) * att[f], &s, &co);
      enc[c * F + f] = round_op(s, precision);
      enc[cos_off + c * F + f] = round_op(co, precision);
    }
  for (int h = 0; h < H; ++h) {
    float acc = 0.f;
    const float* row = M.W1 + (size_t)h * IN;
    for (int k = 0; k < IN; ++k) acc = fmaf(round_op(row[k], precision), enc[k], acc);
    h1[h] = round_op(fmaxf(acc + M.b1[h], 0.f), precision);
  }
  for (int o = 0; o < H; ++o) {
    float acc = 0.f;
    const float* row = M.W2 + (size_t)o * H;
    for (int k = 0; k < H; ++k) acc = fmaf(round_op(row[k], precision), h1[k], acc);
    h2[o] = round_op(fmaxf(acc + M.b2[o], 0.f), precision);
  }
  for (int c = 0; c < 4; ++c) {
    float acc = 0.f;
    const float* row = M.W3 + (size_t)c * H;
    for (int k = 0; k < H; ++k) acc = fmaf(round_op(row[k], precision), h2[k], acc);
    out[c] = acc + M.b3[c];
  }
}

struct Scene {
  const float *rays_o, *rays_d, *pos, *logs, *quats;
  const int32_t *cand, *offsets;
  const float *freq, *att;
  int F;
  const float *W1, *b1, *W2, *b2, *W3, *b3;
  int N, H;
  const float* feat_attr; int feat_slots, C; float beta, temp;
  int Wimg, Himg, TW, TH;
  float thr;
};

inline MlpView mlp_of(const Scene& S, int p) {
  const int H = S.H, IN = 12 * S.F;
  MlpView M;
  M.W1 = S.W1 + (size_t)p * H * IN; M.b1 = S.b1 + (size_t)p * H;
  M.W2 = S.W2 + (size_t)p * H * H;  M.b2 = S.b2 + (size_t)p * H;
  M.W3 = S.W3 + (size_t)p * 4 * H;  M.b3 = S.b3 + (size_t)p * 4;
  M.H = H; M.IN = IN; M.F = S.F;
  return M;
}

// feature accumulate, scannet/cuda/np_tile_kernels.cu:6036-6075
inline void feat_accumulate(const Scene& S, int p, const Prim& P, const Hit& h, float w, float* dst) {
  const int C = S.C, slots = S.feat_slots;
  if (slots <= 1) {
    const float* src = S.feat_attr + (size_t)p * C;
    for (int c = 0; c < C; ++c) dst[c] = fmaf(w, src[c], dst[c]);
    return;
  }
  float g[4];
  tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, S.beta, S.temp, g);
  const float* base = S.feat_attr + (size_t)p * slots * C;
  if (slots == 5) {
    for (int c = 0; c < C; ++c) {
      float mix = base[c];
      mix = fmaf(g[0], base[1 * C + c], mix);
      mix = fmaf(g[1], base[2 * C + c], mix);
      mix = fmaf(g[2], base[3 * C + c], mix);
      mix = fmaf(g[3], base[4 * C + c], mix);
      dst[c] = fmaf(w, mix, dst[c]);
    }
  } else if (slots == 4) {
    for (int c = 0; c < C; ++c) {
      float mix = 0.f;
      mix = fmaf(g[0], base[0 * C + c], mix);
      mix = fmaf(g[1], base[1 * C + c], mix);
      mix = fmaf(g[2], base[2 * C + c], mix);
      mix = fmaf(g[3], base[3 * C + c], mix);
      dst[c] = fmaf(w, mix, dst[c]);
    }
  } else {
    for (int c = 0; c < C; ++c) dst[c] = fmaf(w, base[c], dst[c]);
  }
}

struct PixelState {
  float Cx = 0.f, Cy = 0.f, Cz = 0.f, trans = 1.f, w_acc = 0.f, t_acc = 0.f;
};

// activations + blend, scannet/cuda/np_tile_kernels.cu:2092-2103 (and :5669-5671 for depth)
inline float blend(PixelState& st, const float o[4], float decay, float t) {
  const float sigma_raw = o_softplus(o[3]);
  const float sigma = sigma_raw * decay;
  const float alpha = 1.f - det_exp(-sigma);
  const float w = st.trans * alpha;
  st.w_acc = fmaf(1.f, w, st.w_acc);
  st.t_acc = fmaf(w, t, st.t_acc);
  const float R = o_sigmoid(o[0]), G = o_sigmoid(o[1]), B = o_sigmoid(o[2]);
  st.Cx = fmaf(w, R, st.Cx);
  st.Cy = fmaf(w, G, st.Cy);
  st.Cz = fmaf(w, B, st.Cz);
  st.trans *= (1.f - alpha);
  return w;
}

struct KeyId { float key; int32_t id; };

}  // namespace

// ==========================================================================================
// Exported API (plain C)
// ==========================================================================================

ORACLE_API void mlpsp_oracle_math(int which, const float* x, float* y, float* y2, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    switch (which) {
      case 0: y[i] = det_exp(x[i]); break;
      case 1: det_sincos(x[i], &y[i], &y2[i]); break;
      case 2: y[i] = det_log1p_pos(x[i]); break;
      case 3: y[i] = o_sigmoid(x[i]); break;
      case 4: y[i] = o_softplus(x[i]); break;
      case 5: y[i] = round_bf16(x[i]); break;
      case 6: y[i] = round_f16(x[i]); break;
      default: y[i] = NAN;
    }
  }
}

// out[8] = t, dx, dy, dz, qlx, qly, qlz, decay; returns 1 on hit.
ORACLE_API int mlpsp_oracle_hit(const float* ro, const float* rd, const float* pos, const float* logs,
                                const float* quat, float thr, float* out) {
  const Prim P = load_prim(pos, logs, quat, 0);
  Hit h = {0, 0, 0, 0, 0, 0, 0, 0};
  const bool hit = hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h);
  out[0] = h.t; out[1] = h.dx; out[2] = h.dy; out[3] = h.dz;
  out[4] = h.qlx; out[5] = h.qly; out[6] = h.qlz; out[7] = h.decay;
  return hit ? 1 : 0;
}

ORACLE_API float mlpsp_oracle_key(int family, const float* ro, const float* rd, const float* pos,
                                  const float* logs, const float* quat) {
  const Prim P = load_prim(pos, logs, quat, 0);
  return family == 2 ? key_depth(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P)
                     : key_tstar(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P);
}

ORACLE_API void mlpsp_oracle_gates(const float* ql, const float* logs, float beta, float temp, float* g) {
  tetra_gates(ql[0], ql[1], ql[2], logs[0], logs[1], logs[2], beta, temp, g);
}

// MLP for M records; prim_ids[M] selects the weight block; precision 0 f32, 1 bf16, 2 fp16.
ORACLE_API void mlpsp_oracle_mlp(const float* x6, const int32_t* prim_ids, int64_t M,
                                 const float* freq, const float* att, int F,
                                 const float* W1, const float* b1, const float* W2, const float* b2,
                                 const float* W3, const float* b3, int H, int precision, float* out) {
  Scene S{};
  S.F = F; S.H = H; S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3;
  for (int64_t i = 0; i < M; ++i) {
    const MlpView V = mlp_of(S, prim_ids[i]);
    if (precision == 0) mlp_f32(x6 + i * 6, freq, att, V, out + i * 4);
    else mlp_mixed(x6 + i * 6, freq, att, V, precision, out + i * 4);
  }
}

// Validation, scannet/cuda/np_tile_kernels.cu:4485-4520.  status[0] bit mask (1 offsets, 2 capacity,
// 4 ids), status[1] = largest over-capacity count.
ORACLE_API void mlpsp_oracle_validate(const int32_t* offsets, const int32_t* cand, int num_tiles,
                                      int num_cand, int capacity, int num_prims, int32_t* status) {
  status[0] = 0; status[1] = 0;
  for (int t = 0; t < num_tiles; ++t) {
    const int start = offsets[t], end = offsets[t + 1];
    if (start < 0 || end < start || end > num_cand || (t == 0 && start != 0) ||
        (t == num_tiles - 1 && end != num_cand)) { status[0] |= 1; continue; }
    const int count = end - start;
    if (capacity > 0 && count > capacity) { status[0] |= 2; status[1] = std::max(status[1], count); }
  }
  for (int i = 0; i < num_cand; ++i)
    if (cand[i] < 0 || cand[i] >= num_prims) status[0] |= 4;
}

// ------------------------------------------------------------------------------------------
// Binning.  Legacy rule of scannet/cumodel.py:994-1070 (one camera) and :838-949 (per-tile view).
// view_mats[K][16], proj[16] row-major; tile_view_ids may be null (all tiles use view 0).
// Two-phase: call with cand == nullptr to get counts into offsets[T+1] (exclusive scan applied),
// then with cand to fill.  Returns total pairs.  Within a tile primitive ids ascend.
// ------------------------------------------------------------------------------------------
namespace {
struct Bounds { float minx, maxx, miny, maxy; bool front; };

inline Bounds prim_bounds(const float* V, const float* Pm, const float* pos, const float* logs, int i,
                          float rm, float focal, float Wf, float Hf) {
  const float x = pos[i * 3 + 0], y = pos[i * 3 + 1], z = pos[i * 3 + 2];
  float pv[4];
  for (int k = 0; k < 4; ++k)
    pv[k] = fmaf(V[k * 4 + 0], x, fmaf(V[k * 4 + 1], y, fmaf(V[k * 4 + 2], z, V[k * 4 + 3])));
  const float depth = pv[2];
  Bounds b;
  b.front = depth > 0.001f;
  const float s = fmaxf(fmaxf(det_exp(logs[i * 3 + 0]), det_exp(logs[i * 3 + 1])), det_exp(logs[i * 3 + 2]));
  const float world_radius = s * rm;
  const float pr = (world_radius / (depth + 1e-8f)) * focal;
  float clip[4];
  for (int k = 0; k < 4; ++k)
    clip[k] = fmaf(Pm[k * 4 + 0], pv[0], fmaf(Pm[k * 4 + 1], pv[1], fmaf(Pm[k * 4 + 2], pv[2], Pm[k * 4 + 3] * pv[3])));
  float w = clip[3];
  if (w == 0.f) w = w + 1e-6f;
  const float sx = (((clip[0] / w) + 1.f) * 0.5f) * Wf;
  const float sy = (((clip[1] / w) + 1.f) * 0.5f) * Hf;
  b.minx = sx - pr; b.maxx = sx + pr; b.miny = sy - pr; b.maxy = sy + pr;
  return b;
}
inline bool overlaps(const Bounds& b, int tx, int ty, int ts) {
  // scannet/cumodel.py:1043-1046 (strict inequalities; integer tile edges compared as floats)
  return b.front && b.minx < (float)((tx + 1) * ts) && b.maxx > (float)(tx * ts) &&
         b.miny < (float)((ty + 1) * ts) && b.maxy > (float)(ty * ts);
}
}  // namespace

namespace {
// Tiles t in [lo, hi] are exactly those with mn < (t+1)*ts && mx > t*ts (empty if lo > hi).
inline void tile_range(float mn, float mx, int ts, int nt, int& lo, int& hi) {
  lo = 0; hi = -1;
  if (mn != mn || mx != mx) return;
  const float flo = floorf(mn / (float)ts) - 1.f, fhi = floorf(mx / (float)ts) + 1.f;
  int a = flo < 0.f ? 0 : (flo > (float)(nt - 1) ? nt : (int)flo);
  int b = fhi < 0.f ? -1 : (fhi > (float)(nt - 1) ? nt - 1 : (int)fhi);
  while (a <= b && !(mn < (float)((a + 1) * ts) && mx > (float)(a * ts))) ++a;
  while (b >= a && !(mn < (float)((b + 1) * ts) && mx > (float)(b * ts))) --b;
  lo = a; hi = b;
}
}  // namespace

ORACLE_API int64_t mlpsp_oracle_bin_legacy(const float* pos, const float* logs, int N,
                                           const float* view_mats, int K, const int32_t* tile_view_ids,
                                           const float* proj, int Wimg, int Himg, int ts, float thr,
                                           int32_t* offsets, int32_t* cand) {
  const int ntx = (Wimg + ts - 1) / ts, nty = (Himg + ts - 1) / ts, T = ntx * nty;
  const float rm = sqrtf(-2.0f * logf(thr));
  const float fx = (proj[0] * (float)Wimg) / 2.0f, fy = (proj[5] * (float)Himg) / 2.0f;
  const float focal = (fx + fy) * 0.5f;
  std::vector<int64_t> cursor(T + 1, 0);
  if (cand) for (int t = 0; t <= T; ++t) cursor[t] = offsets[t];
  // primitives outermost and ascending, so every tile's list ascends in primitive id
  for (int i = 0; i < N; ++i) {
    for (int k = 0; k < K; ++k) {
      const Bounds b = prim_bounds(view_mats + k * 16, proj, pos, logs, i, rm, focal, (float)Wimg, (float)Himg);
      if (!b.front) continue;
      int x0, x1, y0, y1;
      tile_range(b.minx, b.maxx, ts, ntx, x0, x1);
      tile_range(b.miny, b.maxy, ts, nty, y0, y1);
      for (int ty = y0; ty <= y1; ++ty)
        for (int tx = x0; tx <= x1; ++tx) {
          const int t = ty * ntx + tx;
          if ((tile_view_ids ? tile_view_ids[t] : 0) != k) continue;   // (without ids every tile uses view 0)
          if (!overlaps(b, tx, ty, ts)) continue;
          if (cand) cand[cursor[t]++] = i; else cursor[t + 1]++;
        }
    }
  }
  if (!cand) {
    for (int t = 0; t < T; ++t) cursor[t + 1] += cursor[t];
    for (int t = 0; t <= T; ++t) offsets[t] = (int32_t)cursor[t];
    return cursor[T];
  }
  return (int64_t)offsets[T];
}

// Dense form of the same rule (one boolean per tile x primitive, as the reference evaluates it):
// used only to pin the sparse form above by brute force on small inputs.  mask[T*N].
ORACLE_API void mlpsp_oracle_bin_legacy_dense(const float* pos, const float* logs, int N,
                                              const float* view_mats, int K, const int32_t* tile_view_ids,
                                              const float* proj, int Wimg, int Himg, int ts, float thr,
                                              uint8_t* mask) {
  const int ntx = (Wimg + ts - 1) / ts, nty = (Himg + ts - 1) / ts, T = ntx * nty;
  const float rm = sqrtf(-2.0f * logf(thr));
  const float fx = (proj[0] * (float)Wimg) / 2.0f, fy = (proj[5] * (float)Himg) / 2.0f;
  const float focal = (fx + fy) * 0.5f;
  for (int t = 0; t < T; ++t) {
    const int v = tile_view_ids ? tile_view_ids[t] : 0;
    for (int i = 0; i < N; ++i) {
      const Bounds b = prim_bounds(view_mats + v * 16, proj, pos, logs, i, rm, focal, (float)Wimg, (float)Himg);
      mask[(size_t)t * N + i] = overlaps(b, t % ntx, t / ntx, ts) ? 1 : 0;
    }
  }
}

// Ray-cone binning, scannet/camera.py:102-146.  Returns -1 if a tile mixes origins, -2 if a cone
// spans >= 90 degrees, otherwise the pair count; same two-phase protocol as above.
ORACLE_API int64_t mlpsp_oracle_bin_raycone(const float* rays_o, const float* rays_d, const float* pos,
                                            const float* logs, int N, int Wimg, int Himg, int ts,
                                            float thr, int32_t* offsets, int32_t* cand) {
  const int ntx = (Wimg + ts - 1) / ts, nty = (Himg + ts - 1) / ts, T = ntx * nty, npx = ts * ts;
  std::vector<float> radius(N);
  const float mult = (float)std::sqrt(-2.0 * std::log((double)thr));
  for (int i = 0; i < N; ++i) {
    const float s = fmaxf(fmaxf(det_exp(logs[i * 3]), det_exp(logs[i * 3 + 1])), det_exp(logs[i * 3 + 2]));
    radius[i] = (s * mult) * (1.f + 1e-5f) + 1e-7f;
  }
  std::vector<int64_t> counts(T + 1, 0);
  int err = 0;
  {
#pragma omp parallel for schedule(dynamic, 8)
    for (int t = 0; t < T; ++t) {
      const int tx = t % ntx, ty = t / ntx;
      std::vector<float> dirs(npx * 3);
      float ax = 0, ay = 0, az = 0;
      const int p0 = std::min(ty * ts, Himg - 1) * Wimg + std::min(tx * ts, Wimg - 1);
      const float ox = rays_o[p0 * 3], oy = rays_o[p0 * 3 + 1], oz = rays_o[p0 * 3 + 2];
      for (int k = 0; k < npx; ++k) {
        const int px = std::min(tx * ts + k % ts, Wimg - 1), py = std::min(ty * ts + k / ts, Himg - 1);
        const int pix = py * Wimg + px;
        if (fabsf(rays_o[pix * 3] - ox) > 1e-6f || fabsf(rays_o[pix * 3 + 1] - oy) > 1e-6f ||
            fabsf(rays_o[pix * 3 + 2] - oz) > 1e-6f) {
#pragma omp atomic write
          err = -1;
        }
        const float dx = rays_d[pix * 3], dy = rays_d[pix * 3 + 1], dz = rays_d[pix * 3 + 2];
        const float n = fmaxf(sqrtf((dx * dx + dy * dy) + dz * dz), 1e-12f);
        dirs[k * 3] = dx / n; dirs[k * 3 + 1] = dy / n; dirs[k * 3 + 2] = dz / n;
        ax += dirs[k * 3]; ay += dirs[k * 3 + 1]; az += dirs[k * 3 + 2];
      }
      ax /= (float)npx; ay /= (float)npx; az /= (float)npx;
      const float an = fmaxf(sqrtf((ax * ax + ay * ay) + az * az), 1e-12f);
      ax /= an; ay /= an; az /= an;
      float cos_t = 1.f;
      for (int k = 0; k < npx; ++k)
        cos_t = fminf(cos_t, (dirs[k * 3] * ax + dirs[k * 3 + 1] * ay) + dirs[k * 3 + 2] * az);
      cos_t = fminf(1.f, fmaxf(-1.f, cos_t));
      if (cos_t <= 0.f) {
#pragma omp atomic write
        err = -2;
      }
      const float sin_t = sqrtf(fmaxf(1.f - cos_t * cos_t, 0.f));
      int64_t w = cand ? offsets[t] : 0;
      for (int i = 0; i < N; ++i) {
        const float ex = pos[i * 3] - ox, ey = pos[i * 3 + 1] - oy, ez = pos[i * 3 + 2] - oz;
        const float dist = sqrtf((ex * ex + ey * ey) + ez * ez);
        const float dc = fmaxf(dist, 1e-20f);
        const float ratio = fminf(1.f, fmaxf(0.f, radius[i] / dc));
        const float cos_b = ((ex * ax + ey * ay) + ez * az) / dc;
        const float bound = cos_t * sqrtf(fmaxf(1.f - ratio * ratio, 0.f)) - sin_t * ratio;
        if (dist <= radius[i] || cos_b >= bound - 2e-6f) {
          if (cand) cand[w] = i;
          ++w;
        }
      }
      counts[t + 1] = cand ? (w - offsets[t]) : w;
    }
  }
  if (err) return err;
  for (int t = 0; t < T; ++t) counts[t + 1] += counts[t];
  if (!cand) for (int t = 0; t <= T; ++t) offsets[t] = (int32_t)counts[t];
  return counts[T];
}

// ------------------------------------------------------------------------------------------
// Per-tile key + stable sort, scannet/cuda/np_tile_kernels.cu:1883-1892, 1929-1990.
// family 1: Mahalanobis t* key; family 2: centre-ray depth key.  Only the first
// min(len, capacity) candidates are sorted (capacity <= 0: all); the rest keep list order.
// sorted_keys may be null.
// ------------------------------------------------------------------------------------------
namespace {
void sort_tile(const Scene& S, int tile, int family, int capacity, std::vector<KeyId>& buf) {
  const int ntx = (S.Wimg + S.TW - 1) / S.TW;
  const int tx = tile % ntx, ty = tile / ntx;
  const int start = S.offsets[tile], end = S.offsets[tile + 1], len = end - start;
  buf.resize(std::max(len, 0));
  if (len <= 0) return;
  const int cxp = std::min(tx * S.TW + (S.TW >> 1), S.Wimg - 1);
  const int cyp = std::min(ty * S.TH + (S.TH >> 1), S.Himg - 1);
  const int pc = cyp * S.Wimg + cxp;
  const float ox = S.rays_o[pc * 3], oy = S.rays_o[pc * 3 + 1], oz = S.rays_o[pc * 3 + 2];
  const float dx = S.rays_d[pc * 3], dy = S.rays_d[pc * 3 + 1], dz = S.rays_d[pc * 3 + 2];
  const int load_n = (capacity > 0 && len > capacity) ? capacity : len;
  for (int i = 0; i < len; ++i) {
    const int p = S.cand[start + i];
    buf[i].id = p;
    if (i < load_n && family != 0) {
      const Prim P = load_prim(S.pos, S.logs, S.quats, p);
      buf[i].key = family == 2 ? key_depth(ox, oy, oz, dx, dy, dz, P) : key_tstar(ox, oy, oz, dx, dy, dz, P);
    } else {
      buf[i].key = 1e30f;
    }
  }
  if (family != 0)
    std::stable_sort(buf.begin(), buf.begin() + load_n,
                     [](const KeyId& a, const KeyId& b) { return a.key < b.key; });
}
}  // namespace

ORACLE_API void mlpsp_oracle_sort_tiles(const float* rays_o, const float* rays_d, const float* pos,
                                        const float* logs, const float* quats, const int32_t* cand,
                                        const int32_t* offsets, int Wimg, int Himg, int TW, int TH,
                                        int family, int capacity, int32_t* sorted_ids, float* sorted_keys) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH;
  const int T = ((Wimg + TW - 1) / TW) * ((Himg + TH - 1) / TH);
#pragma omp parallel
  {
    std::vector<KeyId> buf;
#pragma omp for schedule(dynamic, 8)
    for (int t = 0; t < T; ++t) {
      sort_tile(S, t, family, capacity, buf);
      const int start = offsets[t];
      for (size_t i = 0; i < buf.size(); ++i) {
        sorted_ids[start + i] = buf[i].id;
        if (sorted_keys) sorted_keys[start + i] = buf[i].key;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Tile-centre forward: scannet/cuda/np_tile_kernels.cu:1837-2137 (RGB), :5794-6112 (+feature),
// :5432-5719 (+expected depth, key family 2), rgb_wmma.cuh:75-223 (precision 1/2).
// family 0 consumes the list in the given order (presorted kernel, :4242-4478).
// stats[4] (optional): candidates, tile-primitives processed, tile-primitives with >= 1 hit, hits.
// ------------------------------------------------------------------------------------------
ORACLE_API void mlpsp_oracle_render_tilecenter(
    const float* rays_o, const float* rays_d, const float* pos, const float* logs, const float* quats,
    const int32_t* cand, const int32_t* offsets, const float* freq, const float* att, int F,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int N, int H, const float* feat_attr, int feat_slots, int C, float beta, float temp,
    int Wimg, int Himg, int TW, int TH, float thr, int family, int precision, int capacity,
    float* out_rgb, float* out_alpha, float* out_t, float* out_feat, int64_t* stats, int nthreads) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.freq = freq; S.att = att; S.F = F;
  S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3; S.N = N; S.H = H;
  S.feat_attr = feat_attr; S.feat_slots = feat_slots; S.C = C; S.beta = beta; S.temp = temp;
  S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH; S.thr = thr;
  const int ntx = (Wimg + TW - 1) / TW, nty = (Himg + TH - 1) / TH, T = ntx * nty, npx = TW * TH;
  int64_t s_cand = 0, s_proc = 0, s_proc_hit = 0, s_hits = 0;
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel num_threads(nthreads) reduction(+ : s_cand, s_proc, s_proc_hit, s_hits)
  {
    std::vector<KeyId> buf;
    std::vector<PixelState> st(npx);
    std::vector<int> pixidx(npx);
#pragma omp for schedule(dynamic, 4)
    for (int tile = 0; tile < T; ++tile) {
      const int tx = tile % ntx, ty = tile / ntx;
      int nvalid = 0;
      for (int k = 0; k < npx; ++k) {
        const int x = tx * TW + k % TW, y = ty * TH + k / TW;
        pixidx[k] = (x < Wimg && y < Himg) ? (y * Wimg + x) : -1;
        st[k] = PixelState();
        if (pixidx[k] >= 0) {
          ++nvalid;
          if (out_feat) std::memset(out_feat + (size_t)pixidx[k] * C, 0, sizeof(float) * C);
        }
      }
      sort_tile(S, tile, family, capacity, buf);
      s_cand += (int64_t)buf.size();
      for (size_t i = 0; i < buf.size(); ++i) {
        const int p = buf[i].id;
        if (p < 0 || p >= N) continue;
        const Prim P = load_prim(pos, logs, quats, p);
        const MlpView M = mlp_of(S, p);
        ++s_proc;
        int nhit = 0, nactive = 0;
        for (int k = 0; k < npx; ++k) {
          const int pix = pixidx[k];
          if (pix < 0) continue;
          PixelState& ps = st[k];
          if (ps.trans >= 1e-3f) {
            Hit h;
            const float* ro = rays_o + (size_t)pix * 3;
            const float* rd = rays_d + (size_t)pix * 3;
            if (hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h)) {
              const float x6[6] = {rd[0], rd[1], rd[2], h.dx, h.dy, h.dz};
              float o[4];
              if (precision == 0) mlp_f32(x6, freq, att, M, o);
              else mlp_mixed(x6, freq, att, M, precision, o);
              const float w = blend(ps, o, h.decay, h.t);
              if (out_feat) feat_accumulate(S, p, P, h, w, out_feat + (size_t)pix * C);
              ++nhit;
            }
          }
          if (ps.trans >= 1e-3f) ++nactive;
        }
        s_hits += nhit;
        if (nhit) ++s_proc_hit;
        if (nactive == 0) break;  // block-uniform exit, np_tile_kernels.cu:2115-2116
      }
      for (int k = 0; k < npx; ++k) {
        const int pix = pixidx[k];
        if (pix < 0) continue;
        out_rgb[pix * 3 + 0] = st[k].Cx; out_rgb[pix * 3 + 1] = st[k].Cy; out_rgb[pix * 3 + 2] = st[k].Cz;
        out_alpha[pix] = 1.f - st[k].trans;
        if (out_t) out_t[pix] = st[k].t_acc / (st[k].w_acc > 1e-8f ? st[k].w_acc : 1.f);
      }
      (void)nvalid;
    }
  }
  if (stats) { stats[0] = s_cand; stats[1] = s_proc; stats[2] = s_proc_hit; stats[3] = s_hits; }
}

// ------------------------------------------------------------------------------------------
// Pruning statistics forward: scannet/cuda/np_tile_kernels.cu:2139-2519 (kernel), :5349-5428 (wrapper).
// Plain centre-depth order (:2243-2249), f32.  Per (tile, processed primitive) the block reduces over
// its pixels  w,  max w,  [w > 1e-8],  [w > 0.1] * w * err,  [w > 0.1]  with err the L1 colour error of
// the pixel AFTER this blend step against gt_rgb (:2394-2412), and adds them to five per-primitive
// buffers (:2449-2456).  The reference's reduction and atomic order is unspecified; the sums are kept
// in double here and compared with a tolerance.
// ------------------------------------------------------------------------------------------
ORACLE_API void mlpsp_oracle_render_stats(
    const float* rays_o, const float* rays_d, const float* pos, const float* logs, const float* quats,
    const int32_t* cand, const int32_t* offsets, const float* freq, const float* att, int F,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int N, int H, int Wimg, int Himg, int TW, int TH, float thr, int capacity, const float* gt_rgb,
    float* out_rgb, float* out_alpha, double* sum_w, double* max_w, int64_t* hits, double* sum_werr,
    int64_t* contrib, int nthreads) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.freq = freq; S.att = att; S.F = F;
  S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3; S.N = N; S.H = H;
  S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH; S.thr = thr;
  const int ntx = (Wimg + TW - 1) / TW, nty = (Himg + TH - 1) / TH, T = ntx * nty, npx = TW * TH;
  constexpr float kWEps = 1e-1f;
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel num_threads(nthreads)
  {
    std::vector<KeyId> buf;
    std::vector<PixelState> st(npx);
    std::vector<int> pixidx(npx);
#pragma omp for schedule(dynamic, 4)
    for (int tile = 0; tile < T; ++tile) {
      const int tx = tile % ntx, ty = tile / ntx;
      for (int k = 0; k < npx; ++k) {
        const int x = tx * TW + k % TW, y = ty * TH + k / TW;
        pixidx[k] = (x < Wimg && y < Himg) ? (y * Wimg + x) : -1;
        st[k] = PixelState();
      }
      sort_tile(S, tile, 2, capacity, buf);
      for (size_t i = 0; i < buf.size(); ++i) {
        const int p = buf[i].id;
        if (p < 0 || p >= N) continue;
        const Prim P = load_prim(pos, logs, quats, p);
        const MlpView M = mlp_of(S, p);
        double t_sum = 0.0, t_werr = 0.0;
        float t_max = 0.f;
        int64_t t_hits = 0, t_contrib = 0;
        int nactive = 0;
        for (int k = 0; k < npx; ++k) {
          const int pix = pixidx[k];
          if (pix < 0) continue;
          PixelState& ps = st[k];
          if (ps.trans >= 1e-3f) {
            Hit h;
            const float* ro = rays_o + (size_t)pix * 3;
            const float* rd = rays_d + (size_t)pix * 3;
            if (hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h)) {
              const float x6[6] = {rd[0], rd[1], rd[2], h.dx, h.dy, h.dz};
              float o[4];
              mlp_f32(x6, freq, att, M, o);
              const float w = blend(ps, o, h.decay, h.t);
              const float* gt = gt_rgb + (size_t)pix * 3;
              const float err = (std::fabs(ps.Cx - gt[0]) + std::fabs(ps.Cy - gt[1])) + std::fabs(ps.Cz - gt[2]);
              t_sum += (double)w;
              t_max = w > t_max ? w : t_max;
              t_hits += (w > 1e-8f) ? 1 : 0;
              if (w > kWEps) {
                t_werr += (double)(w * err);
                ++t_contrib;
              }
            }
          }
          if (ps.trans >= 1e-3f) ++nactive;
        }
#pragma omp atomic
        sum_w[p] += t_sum;
#pragma omp atomic
        sum_werr[p] += t_werr;
#pragma omp atomic
        hits[p] += t_hits;
#pragma omp atomic
        contrib[p] += t_contrib;
#pragma omp critical(mlpsp_stat_max)
        { if ((double)t_max > max_w[p]) max_w[p] = (double)t_max; }
        if (nactive == 0) break;
      }
      for (int k = 0; k < npx; ++k) {
        const int pix = pixidx[k];
        if (pix < 0) continue;
        out_rgb[pix * 3 + 0] = st[k].Cx; out_rgb[pix * 3 + 1] = st[k].Cy; out_rgb[pix * 3 + 2] = st[k].Cz;
        out_alpha[pix] = 1.f - st[k].trans;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Training-records forward: scannet/cuda/np_tile_kernels.cu:2925-3206 (modes 1 and 3), wrapper
// :6897-6998.  t* order, f32, hidden <= 32.  Per pixel, for every hit taken while the pixel is live
// (T >= 1e-3) and has fewer than max_hits records: id, x6 = (ray direction, world offset), ReLU masks,
// raw = (R, G, B, sigma_raw, T before the hit, alpha, decay, sigma logit), gates; rgb and alpha are the
// composite of those records.  A live pixel that already holds max_hits records sets *overflow (the
// reference then raises "hit capacity", :3166-3168, 4601-4609).
// Two-phase: ids == nullptr -> counts[B] only; else records are written at offsets[pix] + k.
// ------------------------------------------------------------------------------------------
ORACLE_API void mlpsp_oracle_records(
    const float* rays_o, const float* rays_d, const float* pos, const float* logs, const float* quats,
    const int32_t* cand, const int32_t* offsets, const float* freq, const float* att, int F,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int N, int H, int Wimg, int Himg, int TW, int TH, float thr, int capacity, int max_hits, float beta, float temp,
    int32_t* counts, int32_t* overflow, const int64_t* rec_offsets, int32_t* ids, float* x6_out, int32_t* masks_out,
    float* raw_out, float* gates_out, float* out_rgb, float* out_alpha, int nthreads) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.freq = freq; S.att = att; S.F = F;
  S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3; S.N = N; S.H = H;
  S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH; S.thr = thr;
  const int ntx = (Wimg + TW - 1) / TW, nty = (Himg + TH - 1) / TH, T = ntx * nty, npx = TW * TH;
  int ovf = 0;
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel num_threads(nthreads) reduction(| : ovf)
  {
    std::vector<KeyId> buf;
    std::vector<float> trans(npx), cr(npx), cg(npx), cb(npx);
    std::vector<int> used(npx), pixidx(npx);
#pragma omp for schedule(dynamic, 4)
    for (int tile = 0; tile < T; ++tile) {
      const int tx = tile % ntx, ty = tile / ntx;
      for (int k = 0; k < npx; ++k) {
        const int x = tx * TW + k % TW, y = ty * TH + k / TW;
        pixidx[k] = (x < Wimg && y < Himg) ? (y * Wimg + x) : -1;
        trans[k] = 1.f; cr[k] = cg[k] = cb[k] = 0.f; used[k] = 0;
      }
      sort_tile(S, tile, 1, capacity, buf);
      for (size_t i = 0; i < buf.size(); ++i) {
        const int p = buf[i].id;
        int nactive = 0;
        if (p >= 0 && p < N) {
          const Prim P = load_prim(pos, logs, quats, p);
          const MlpView M = mlp_of(S, p);
          for (int k = 0; k < npx; ++k) {
            const int pix = pixidx[k];
            if (pix < 0 || trans[k] < 1e-3f || used[k] >= max_hits) continue;
            Hit h;
            const float* ro = rays_o + (size_t)pix * 3;
            const float* rd = rays_d + (size_t)pix * 3;
            if (!hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h)) continue;
            const float v6[6] = {rd[0], rd[1], rd[2], h.dx, h.dy, h.dz};
            float o[4];
            uint32_t mk[2];
            mlp_f32_records(v6, freq, att, M, o, mk);
            const float R = o_sigmoid(o[0]), G = o_sigmoid(o[1]), Bc = o_sigmoid(o[2]);
            const float sigma_raw = o_softplus(o[3]);
            const float sigma = sigma_raw * h.decay;
            const float alpha = 1.f - det_exp(-sigma);
            if (ids) {
              const int64_t r = rec_offsets[pix] + used[k];
              ids[r] = p;
              for (int c = 0; c < 6; ++c) x6_out[r * 6 + c] = v6[c];
              masks_out[r * 2] = (int32_t)mk[0];
              masks_out[r * 2 + 1] = (int32_t)mk[1];
              float* raw = raw_out + r * 8;
              raw[0] = R; raw[1] = G; raw[2] = Bc; raw[3] = sigma_raw;
              raw[4] = trans[k]; raw[5] = alpha; raw[6] = h.decay; raw[7] = o[3];
              tetra_gates(h.qlx, h.qly, h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gates_out + r * 4);
              const float weight = trans[k] * alpha;
              cr[k] = fmaf(weight, R, cr[k]);
              cg[k] = fmaf(weight, G, cg[k]);
              cb[k] = fmaf(weight, Bc, cb[k]);
            }
            trans[k] *= (1.f - alpha);
            ++used[k];
          }
        }
        for (int k = 0; k < npx; ++k) {
          if (pixidx[k] < 0 || trans[k] < 1e-3f) continue;
          ++nactive;
          if (used[k] >= max_hits) ovf |= 1;
        }
        if (nactive == 0) break;
      }
      for (int k = 0; k < npx; ++k) {
        const int pix = pixidx[k];
        if (pix < 0) continue;
        if (!ids) {
          counts[pix] = used[k];
        } else {
          out_rgb[pix * 3 + 0] = cr[k]; out_rgb[pix * 3 + 1] = cg[k]; out_rgb[pix * 3 + 2] = cb[k];
          out_alpha[pix] = 1.f - trans[k];
        }
      }
    }
  }
  if (overflow) *overflow = ovf;
}

// ------------------------------------------------------------------------------------------
// Per-pixel-order forward: scannet/cuda/np_tile_kernels.cu:715-926 (RGB), :929-1208 (+feature).
// Returns 1 if some pixel met a 257th hit (the reference then raises), else 0.
// ------------------------------------------------------------------------------------------
ORACLE_API int mlpsp_oracle_render_per_pixel(
    const float* rays_o, const float* rays_d, const float* pos, const float* logs, const float* quats,
    const int32_t* cand, const int32_t* offsets, const float* freq, const float* att, int F,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int N, int H, const float* feat_attr, int feat_slots, int C, float beta, float temp,
    int Wimg, int Himg, int TW, int TH, float thr,
    float* out_rgb, float* out_alpha, float* out_feat, int nthreads) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.freq = freq; S.att = att; S.F = F;
  S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3; S.N = N; S.H = H;
  S.feat_attr = feat_attr; S.feat_slots = feat_slots; S.C = C; S.beta = beta; S.temp = temp;
  S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH; S.thr = thr;
  const int ntx = (Wimg + TW - 1) / TW;
  constexpr int MAXI = 256;
  int overflow = 0;
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 64) num_threads(nthreads) reduction(| : overflow)
  for (int pix = 0; pix < Wimg * Himg; ++pix) {
    const int x = pix % Wimg, y = pix / Wimg;
    const int tile = (y / TH) * ntx + (x / TW);
    const float* ro = rays_o + (size_t)pix * 3;
    const float* rd = rays_d + (size_t)pix * 3;
    struct Rec { Hit h; int p; };
    std::vector<Rec> recs;
    recs.reserve(64);
    for (int k = offsets[tile]; k < offsets[tile + 1]; ++k) {
      const int p = cand[k];
      const Prim P = load_prim(pos, logs, quats, p);
      Hit h;
      if (hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h)) {
        if ((int)recs.size() < MAXI) recs.push_back(Rec{h, p});
        else { overflow |= 1; break; }
      }
    }
    if (out_feat) std::memset(out_feat + (size_t)pix * C, 0, sizeof(float) * C);
    if (recs.empty()) {
      out_rgb[pix * 3] = out_rgb[pix * 3 + 1] = out_rgb[pix * 3 + 2] = 0.f;
      out_alpha[pix] = 0.f;
      continue;
    }
    // insertion sort with strict '>' (np_tile_kernels.cu:822-843) == stable sort by t
    std::stable_sort(recs.begin(), recs.end(), [](const Rec& a, const Rec& b) { return a.h.t < b.h.t; });
    PixelState ps;
    for (const Rec& r : recs) {
      const float x6[6] = {rd[0], rd[1], rd[2], r.h.dx, r.h.dy, r.h.dz};
      float o[4];
      mlp_f32(x6, freq, att, mlp_of(S, r.p), o);
      const float w = blend(ps, o, r.h.decay, r.h.t);
      if (out_feat) {
        const Prim P = load_prim(pos, logs, quats, r.p);
        feat_accumulate(S, r.p, P, r.h, w, out_feat + (size_t)pix * C);
      }
      if (ps.trans < 1e-3f) break;
    }
    out_rgb[pix * 3] = ps.Cx; out_rgb[pix * 3 + 1] = ps.Cy; out_rgb[pix * 3 + 2] = ps.Cz;
    out_alpha[pix] = 1.f - ps.trans;
  }
  return overflow;
}

// ------------------------------------------------------------------------------------------
// Training records in PER-PIXEL order: what render_tiles_backward_count_per_pixel / _emit_per_pixel traverse
// (scannet/cuda/np_tile_kernels.cu:1211-1836: gather <= 256 hits in list order, stable sort by the pixel's own t,
// blend until T < 1e-3), with the record schema of the tile-centre records (:3138-3154) and the record kernels'
// MLP arithmetic (mlp_eval_rgb_sigma).  Two-phase: ids == nullptr -> counts[B]; else records at
// rec_offsets[pix] + k and the image.  Returns 1 if some pixel met a 257th hit.
// ------------------------------------------------------------------------------------------
ORACLE_API int mlpsp_oracle_records_per_pixel(
    const float* rays_o, const float* rays_d, const float* pos, const float* logs, const float* quats,
    const int32_t* cand, const int32_t* offsets, const float* freq, const float* att, int F,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int N, int H, int Wimg, int Himg, int TW, int TH, float thr, float beta, float temp,
    int32_t* counts, const int64_t* rec_offsets, int32_t* ids, float* x6_out, int32_t* masks_out,
    float* raw_out, float* gates_out, float* out_rgb, float* out_alpha, int nthreads) {
  Scene S{};
  S.rays_o = rays_o; S.rays_d = rays_d; S.pos = pos; S.logs = logs; S.quats = quats;
  S.cand = cand; S.offsets = offsets; S.freq = freq; S.att = att; S.F = F;
  S.W1 = W1; S.b1 = b1; S.W2 = W2; S.b2 = b2; S.W3 = W3; S.b3 = b3; S.N = N; S.H = H;
  S.Wimg = Wimg; S.Himg = Himg; S.TW = TW; S.TH = TH; S.thr = thr;
  const int ntx = (Wimg + TW - 1) / TW;
  constexpr int MAXI = 256;
  int overflow = 0;
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 64) num_threads(nthreads) reduction(| : overflow)
  for (int pix = 0; pix < Wimg * Himg; ++pix) {
    const int x = pix % Wimg, y = pix / Wimg;
    const int tile = (y / TH) * ntx + (x / TW);
    const float* ro = rays_o + (size_t)pix * 3;
    const float* rd = rays_d + (size_t)pix * 3;
    struct Rec { Hit h; int p; };
    std::vector<Rec> recs;
    for (int k = offsets[tile]; k < offsets[tile + 1]; ++k) {
      const int p = cand[k];
      const Prim P = load_prim(pos, logs, quats, p);
      Hit h;
      if (hit_rot(ro[0], ro[1], ro[2], rd[0], rd[1], rd[2], P, thr, h)) {
        if ((int)recs.size() < MAXI) recs.push_back(Rec{h, p});
        else { overflow |= 1; break; }
      }
    }
    std::stable_sort(recs.begin(), recs.end(), [](const Rec& a, const Rec& b) { return a.h.t < b.h.t; });
    float trans = 1.f, cr = 0.f, cg = 0.f, cb = 0.f;
    int used = 0;
    for (const Rec& rec : recs) {
      if (trans < 1e-3f) break;
      const float v6[6] = {rd[0], rd[1], rd[2], rec.h.dx, rec.h.dy, rec.h.dz};
      float o[4];
      uint32_t mk[2];
      mlp_f32_records(v6, freq, att, mlp_of(S, rec.p), o, mk);
      const float R = o_sigmoid(o[0]), G = o_sigmoid(o[1]), Bc = o_sigmoid(o[2]);
      const float sigma_raw = o_softplus(o[3]);
      const float alpha = 1.f - det_exp(-(sigma_raw * rec.h.decay));
      if (ids) {
        const int64_t r = rec_offsets[pix] + used;
        ids[r] = rec.p;
        for (int c = 0; c < 6; ++c) x6_out[r * 6 + c] = v6[c];
        masks_out[r * 2] = (int32_t)mk[0];
        masks_out[r * 2 + 1] = (int32_t)mk[1];
        float* raw = raw_out + r * 8;
        raw[0] = R; raw[1] = G; raw[2] = Bc; raw[3] = sigma_raw;
        raw[4] = trans; raw[5] = alpha; raw[6] = rec.h.decay; raw[7] = o[3];
        const Prim P = load_prim(pos, logs, quats, rec.p);
        tetra_gates(rec.h.qlx, rec.h.qly, rec.h.qlz, P.lgx, P.lgy, P.lgz, beta, temp, gates_out + r * 4);
        const float weight = trans * alpha;
        cr = fmaf(weight, R, cr);
        cg = fmaf(weight, G, cg);
        cb = fmaf(weight, Bc, cb);
      }
      trans *= (1.f - alpha);
      ++used;
    }
    if (!ids) {
      counts[pix] = used;
    } else {
      out_rgb[pix * 3] = cr; out_rgb[pix * 3 + 1] = cg; out_rgb[pix * 3 + 2] = cb;
      out_alpha[pix] = 1.f - trans;
    }
  }
  return overflow;
}

// ------------------------------------------------------------------------------------------
// Reverse compositing over saved forward records (scannet/cuda/primitive_records.cuh:3-46): per pixel, last
// record first, the adjoint d4 of the four pre-activation MLP outputs of every record and the geometry
// gradients that flow through the Gaussian falloff `decay` (the hit offset x6[3:6] is treated as given):
// grad of positions, log-scales and quaternions, accumulated per primitive.  Here sequential (pixels
// ascending), so the sums have one fixed order; the device kernels add with atomics in any order.
// quaternion gradient: chain rule through the rotation matrix, np_tile_kernels.cu:439-479.
// ------------------------------------------------------------------------------------------
ORACLE_API void mlpsp_oracle_records_reverse(const int32_t* ids, const int64_t* offsets, const float* x6,
                                             const float* raw, const float* logs, const float* quats,
                                             const float* grgb, const float* gt, int64_t pixels, float* d4,
                                             float* gp, float* gs, float* gq) {
  for (int64_t pix = 0; pix < pixels; ++pix) {
    float next = gt[pix];
    const float g0 = grgb[pix * 3], g1 = grgb[pix * 3 + 1], g2 = grgb[pix * 3 + 2];
    for (int64_t r = offsets[pix + 1] - 1; r >= offsets[pix]; --r) {
      const int p = ids[r];
      const float* v = raw + r * 8;
      const float R = v[0], G = v[1], B = v[2], sigma_raw = v[3], trans = v[4], alpha = v[5], decay = v[6];
      const float dotg = (g0 * R + g1 * G) + g2 * B;
      const float grad_alpha = trans * (dotg - next);
      next = next * (1.f - alpha) + dotg * alpha;
      const float grad_sigma = grad_alpha * det_exp(-sigma_raw * decay);
      const float grad_decay = grad_sigma * sigma_raw;
      d4[r * 4 + 0] = g0 * (trans * alpha) * R * (1.f - R);
      d4[r * 4 + 1] = g1 * (trans * alpha) * G * (1.f - G);
      d4[r * 4 + 2] = g2 * (trans * alpha) * B * (1.f - B);
      d4[r * 4 + 3] = grad_sigma * decay * o_sigmoid(v[7]);
      const float dx = x6[r * 6 + 3], dy = x6[r * 6 + 4], dz = x6[r * 6 + 5];
      const float qw = quats[p * 4], qx = quats[p * 4 + 1], qy = quats[p * 4 + 2], qz = quats[p * 4 + 3];
      const V3 q = quat_rotate_conj(qw, qx, qy, qz, V3{dx, dy, dz});
      const float mx = det_exp(-2.f * logs[p * 3]), my = det_exp(-2.f * logs[p * 3 + 1]),
                  mz = det_exp(-2.f * logs[p * 3 + 2]);
      const float gx = -grad_decay * decay * mx * q.x;
      const float gy = -grad_decay * decay * my * q.y;
      const float gz = -grad_decay * decay * mz * q.z;
      const V3 gd = quat_rotate(qw, qx, qy, qz, V3{gx, gy, gz});
      gp[p * 3] += gd.x;
      gp[p * 3 + 1] += gd.y;
      gp[p * 3 + 2] += gd.z;
      gs[p * 3] += grad_decay * decay * mx * q.x * q.x;
      gs[p * 3 + 1] += grad_decay * decay * my * q.y * q.y;
      gs[p * 3 + 2] += grad_decay * decay * mz * q.z * q.z;
      const float r00 = dx * gx, r01 = dx * gy, r02 = dx * gz, r10 = dy * gx, r11 = dy * gy, r12 = dy * gz,
                  r20 = dz * gx, r21 = dz * gy, r22 = dz * gz;
      gq[p * 4] += r01 * (-2.f * qz) + r02 * (2.f * qy) + r10 * (2.f * qz) + r12 * (-2.f * qx) + r20 * (-2.f * qy) +
                   r21 * (2.f * qx);
      gq[p * 4 + 1] += r01 * (2.f * qy) + r02 * (2.f * qz) + r10 * (2.f * qy) + r11 * (-4.f * qx) + r12 * (-2.f * qw) +
                       r20 * (2.f * qz) + r21 * (2.f * qw) + r22 * (-4.f * qx);
      gq[p * 4 + 2] += r00 * (-4.f * qy) + r01 * (2.f * qx) + r02 * (2.f * qw) + r10 * (2.f * qx) + r12 * (2.f * qz) +
                       r20 * (-2.f * qw) + r21 * (2.f * qz) + r22 * (-4.f * qy);
      gq[p * 4 + 3] += r00 * (-4.f * qz) + r01 * (-2.f * qw) + r02 * (2.f * qx) + r10 * (2.f * qw) + r11 * (-4.f * qz) +
                       r12 * (2.f * qy) + r20 * (2.f * qx) + r21 * (2.f * qy);
    }
  }
}

ORACLE_API int mlpsp_oracle_num_threads(void) { return omp_get_max_threads(); }
