// libmlpsp_hip: ray-cone tile binning for cameras whose rays are not a centred pinhole.
//
// Rule of scannet/camera.py:102-146: a tile's rays share one origin and lie inside a cone (axis =
// normalised mean direction, half-angle = largest deviation); a primitive is kept if the sphere
// enclosing its threshold ellipsoid meets the cone.  The reference evaluates [128 tiles x N]
// tensor blocks; here one thread builds each tile's cone, then one wavefront per tile streams the
// primitives 64 at a time (position + radius = 16 B per test, coalesced), counting with a ballot
// and, after a scan, writing survivors at ballot-prefix positions, i.e. in ascending id order.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"

#include <math.h>

namespace mlpsp {

struct __attribute__((aligned(32))) TileCone {
  float ox, oy, oz, cos_t, ax, ay, az, sin_t;
};

__global__ __launch_bounds__(256) void raycone_tiles_kernel(const float* __restrict__ rays_o,
                                                            const float* __restrict__ rays_d, int W, int H, int ts,
                                                            int ntx, int T, TileCone* __restrict__ cones,
                                                            int32_t* __restrict__ flags) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const int tx = t % ntx, ty = t / ntx, npx = ts * ts;
  const int p0 = min(ty * ts, H - 1) * W + min(tx * ts, W - 1);
  const float ox = rays_o[p0 * 3], oy = rays_o[p0 * 3 + 1], oz = rays_o[p0 * 3 + 2];
  float ax = 0.f, ay = 0.f, az = 0.f;
  bool mixed = false;
  for (int k = 0; k < npx; ++k) {
    const int pix = min(ty * ts + k / ts, H - 1) * W + min(tx * ts + k % ts, W - 1);
    mixed |= fabsf(rays_o[pix * 3] - ox) > 1e-6f || fabsf(rays_o[pix * 3 + 1] - oy) > 1e-6f ||
             fabsf(rays_o[pix * 3 + 2] - oz) > 1e-6f;
    const float dx = rays_d[pix * 3], dy = rays_d[pix * 3 + 1], dz = rays_d[pix * 3 + 2];
    const float n = fmaxf(sqrtf((dx * dx + dy * dy) + dz * dz), 1e-12f);
    ax += dx / n;
    ay += dy / n;
    az += dz / n;
  }
  ax /= (float)npx;
  ay /= (float)npx;
  az /= (float)npx;
  const float an = fmaxf(sqrtf((ax * ax + ay * ay) + az * az), 1e-12f);
  ax /= an;
  ay /= an;
  az /= an;
  float cos_t = 1.f;
  for (int k = 0; k < npx; ++k) {
    const int pix = min(ty * ts + k / ts, H - 1) * W + min(tx * ts + k % ts, W - 1);
    const float dx = rays_d[pix * 3], dy = rays_d[pix * 3 + 1], dz = rays_d[pix * 3 + 2];
    const float n = fmaxf(sqrtf((dx * dx + dy * dy) + dz * dz), 1e-12f);
    cos_t = fminf(cos_t, ((dx / n) * ax + (dy / n) * ay) + (dz / n) * az);
  }
  cos_t = fminf(1.f, fmaxf(-1.f, cos_t));
  if (mixed) atomicOr(flags, 1);
  if (cos_t <= 0.f) atomicOr(flags, 2);
  TileCone c;
  c.ox = ox; c.oy = oy; c.oz = oz; c.cos_t = cos_t;
  c.ax = ax; c.ay = ay; c.az = az;
  c.sin_t = sqrtf(fmaxf(1.f - cos_t * cos_t, 0.f));
  cones[t] = c;
}

// (x, y, z, radius) per primitive; radius = max_k exp(log_s_k) * mult * (1 + 1e-5) + 1e-7
__global__ __launch_bounds__(256) void raycone_spheres_kernel(const float* __restrict__ pos,
                                                              const float* __restrict__ logs, int N, float mult,
                                                              float4* __restrict__ spheres) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float s = fmaxf(fmaxf(det_exp(logs[i * 3]), det_exp(logs[i * 3 + 1])), det_exp(logs[i * 3 + 2]));
  spheres[i] = make_float4(pos[i * 3], pos[i * 3 + 1], pos[i * 3 + 2], (s * mult) * (1.f + 1e-5f) + 1e-7f);
}

template <bool FILL>
__global__ __launch_bounds__(256) void raycone_bin_kernel(const TileCone* __restrict__ cones,
                                                          const float4* __restrict__ spheres, int N, int T,
                                                          int32_t* __restrict__ tile_offsets,
                                                          int32_t* __restrict__ cand) {
  const int tile = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (tile >= T) return;
  const TileCone c = cones[tile];
  int running = FILL ? tile_offsets[tile] : 0;
  for (int base = 0; base < N; base += 64) {
    const int i = base + lane;
    bool keep = false;
    if (i < N) {
      const float4 s = spheres[i];
      const float ex = s.x - c.ox, ey = s.y - c.oy, ez = s.z - c.oz;
      const float dist = sqrtf((ex * ex + ey * ey) + ez * ez);
      const float dc = fmaxf(dist, 1e-20f);
      const float ratio = fminf(1.f, fmaxf(0.f, s.w / dc));
      const float cos_b = ((ex * c.ax + ey * c.ay) + ez * c.az) / dc;
      const float bound = c.cos_t * sqrtf(fmaxf(1.f - ratio * ratio, 0.f)) - c.sin_t * ratio;
      keep = (dist <= s.w) || (cos_b >= bound - 2e-6f);
    }
    const unsigned long long m = __ballot(keep);
    if (FILL && keep)
      cand[running + __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u))] = i;
    running += __popcll(m);
  }
  if (!FILL && lane == 0) tile_offsets[tile] = running;
}

__global__ __launch_bounds__(1024) void raycone_scan_kernel(int32_t* __restrict__ data, int n,
                                                            long long* __restrict__ total) {
  __shared__ long long s_part[1024];
  const int t = threadIdx.x;
  const int per = (n + 1023) / 1024;
  const int lo = min(t * per, n), hi = min(lo + per, n);
  long long sum = 0;
  for (int i = lo; i < hi; ++i) sum += data[i];
  s_part[t] = sum;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const long long v = (t >= d) ? s_part[t - d] : 0;
    __syncthreads();
    s_part[t] += v;
    __syncthreads();
  }
  long long run = s_part[t] - sum;
  for (int i = lo; i < hi; ++i) {
    const int v = data[i];
    data[i] = (int32_t)run;
    run += v;
  }
  if (t == 1023) {
    data[n] = (int32_t)s_part[1023];
    *total = s_part[1023];
  }
}

struct RayconeScratch {
  long long* total;
  int32_t* flags;
  TileCone* cones;
  float4* spheres;
};
inline size_t rc_align(size_t x) { return (x + 255) & ~(size_t)255; }
inline RayconeScratch rc_carve(void* base, int T) {
  char* p = static_cast<char*>(base);
  RayconeScratch s;
  s.total = reinterpret_cast<long long*>(p);
  s.flags = reinterpret_cast<int32_t*>(p + 64);
  s.cones = reinterpret_cast<TileCone*>(p + 256);
  s.spheres = reinterpret_cast<float4*>(p + 256 + rc_align((size_t)T * sizeof(TileCone)));
  return s;
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API size_t mlpsp_bin_raycone_scratch_bytes(int num_primitives, int width, int height, int tile) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (T <= 0 || num_primitives < 0) return 0;
  return 256 + rc_align((size_t)T * sizeof(TileCone)) + rc_align((size_t)num_primitives * sizeof(float4)) + 256;
}

MLPSP_API int mlpsp_bin_raycone_count(const float* rays_o_dev, const float* rays_d_dev, const float* positions_dev,
                                      const float* log_scales_dev, int num_primitives, int width, int height,
                                      int tile, float threshold, void* scratch_dev, size_t scratch_bytes,
                                      int32_t* tile_offsets_dev, int64_t* num_pairs_out, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (T <= 0 || T > 2147483647LL || num_primitives < 0 || !rays_o_dev || !rays_d_dev || !scratch_dev ||
      !tile_offsets_dev || !num_pairs_out || tile > 16)
    return MLPSP_E_ARGUMENT;
  if (!(threshold > 0.f && threshold < 1.f)) return MLPSP_E_ARGUMENT;
  if (scratch_bytes < mlpsp_bin_raycone_scratch_bytes(num_primitives, width, height, tile)) return MLPSP_E_SCRATCH;
  hipStream_t s = (hipStream_t)stream;
  const RayconeScratch sc = rc_carve(scratch_dev, (int)T);
  const int ntx = ceil_div(width, tile);
  const float mult = (float)sqrt(-2.0 * log((double)threshold));
  MLPSP_HIP_TRY(hipMemsetAsync(scratch_dev, 0, 256, s));
  hipLaunchKernelGGL(raycone_tiles_kernel, dim3(ceil_div((int)T, 256)), dim3(256), 0, s, rays_o_dev, rays_d_dev, width,
                     height, tile, ntx, (int)T, sc.cones, sc.flags);
  MLPSP_LAUNCH_CHECK();
  if (num_primitives > 0) {
    hipLaunchKernelGGL(raycone_spheres_kernel, dim3(ceil_div(num_primitives, 256)), dim3(256), 0, s, positions_dev,
                       log_scales_dev, num_primitives, mult, sc.spheres);
    MLPSP_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL((raycone_bin_kernel<false>), dim3(ceil_div((int)T, 4)), dim3(256), 0, s, sc.cones, sc.spheres,
                     num_primitives, (int)T, tile_offsets_dev, (int32_t*)nullptr);
  MLPSP_LAUNCH_CHECK();
  hipLaunchKernelGGL(raycone_scan_kernel, dim3(1), dim3(1024), 0, s, tile_offsets_dev, (int)T, sc.total);
  MLPSP_LAUNCH_CHECK();
  struct { long long total; long long pad[7]; int32_t flags; } host = {};
  MLPSP_HIP_TRY(hipMemcpyAsync(&host, scratch_dev, 68, hipMemcpyDeviceToHost, s));
  MLPSP_HIP_TRY(hipStreamSynchronize(s));
  if (host.flags & 1) return MLPSP_E_MIXED_ORIGINS;
  if (host.flags & 2) return MLPSP_E_WIDE_CONE;
  if (host.total > 2147483647LL) return MLPSP_E_ARGUMENT;
  *num_pairs_out = host.total;
  return MLPSP_OK;
}

MLPSP_API int mlpsp_bin_raycone_fill(int num_primitives, int width, int height, int tile, const void* scratch_dev,
                                     size_t scratch_bytes, const int32_t* tile_offsets_dev, int32_t* candidates_dev,
                                     mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile, tile);
  if (T <= 0 || num_primitives < 0 || !scratch_dev || !tile_offsets_dev) return MLPSP_E_ARGUMENT;
  if (scratch_bytes < mlpsp_bin_raycone_scratch_bytes(num_primitives, width, height, tile)) return MLPSP_E_SCRATCH;
  if (num_primitives == 0) return MLPSP_OK;
  if (!candidates_dev) return MLPSP_E_ARGUMENT;
  const RayconeScratch sc = rc_carve(const_cast<void*>(scratch_dev), (int)T);
  hipLaunchKernelGGL((raycone_bin_kernel<true>), dim3(ceil_div((int)T, 4)), dim3(256), 0, (hipStream_t)stream, sc.cones,
                     sc.spheres, num_primitives, (int)T, const_cast<int32_t*>(tile_offsets_dev), candidates_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
