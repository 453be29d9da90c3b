// libmlpsp_hip: primitive preparation, tile-list validation and the per-tile depth-key sort.
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"
#include "mlpsp_sort_tile.hpp"

#include <math.h>

namespace mlpsp {

// ---------------------------------------------------------------------------------------------
// prepare: [N,3]+[N,3]+[N,4] -> one 128-byte record per primitive (HBM-bound: 40 B in, 128 B out)
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void prepare_primitives_kernel(const float* __restrict__ pos,
                                                                 const float* __restrict__ logs,
                                                                 const float* __restrict__ quats, int N,
                                                                 PrimRecord* __restrict__ out) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= N) return;
  PrimRecord r;
  r.cx = pos[p * 3 + 0];
  r.cy = pos[p * 3 + 1];
  r.cz = pos[p * 3 + 2];
  r.lgx = logs[p * 3 + 0];
  r.lgy = logs[p * 3 + 1];
  r.lgz = logs[p * 3 + 2];
  r.qw = quats[p * 4 + 0];
  r.qx = quats[p * 4 + 1];
  r.qy = quats[p * 4 + 2];
  r.qz = quats[p * 4 + 3];
  r.mx = det_exp(-2.f * r.lgx);
  r.my = det_exp(-2.f * r.lgy);
  r.mz = det_exp(-2.f * r.lgz);
  r.s2x = det_exp(2.f * r.lgx);
  r.s2y = det_exp(2.f * r.lgy);
  r.s2z = det_exp(2.f * r.lgz);
  float4* dst = reinterpret_cast<float4*>(out + p);
  dst[0] = make_float4(r.cx, r.cy, r.cz, r.mx);
  dst[1] = make_float4(r.my, r.mz, r.qw, r.qx);
  dst[2] = make_float4(r.qy, r.qz, r.lgx, r.lgy);
  dst[3] = make_float4(r.lgz, r.s2x, r.s2y, r.s2z);
  // second half: centre, then R(q)^T of the unit quaternion row by row, row k scaled by exp(-log_s[k])
  const float w = r.qw, x = r.qx, y = r.qy, z = r.qz;
  const float ix = det_exp(-r.lgx), iy = det_exp(-r.lgy), iz = det_exp(-r.lgz);
  dst[4] = make_float4(r.cx, r.cy, r.cz, ix * (1.f - 2.f * (y * y + z * z)));
  dst[5] = make_float4(ix * (2.f * (x * y + w * z)), ix * (2.f * (x * z - w * y)), iy * (2.f * (x * y - w * z)),
                       iy * (1.f - 2.f * (x * x + z * z)));
  dst[6] = make_float4(iy * (2.f * (y * z + w * x)), iz * (2.f * (x * z + w * y)), iz * (2.f * (y * z - w * x)),
                       iz * (1.f - 2.f * (x * x + y * y)));
  dst[7] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// ---------------------------------------------------------------------------------------------
// validate (np_tile_kernels.cu:4485-4520): grid-stride over tiles, then over candidates
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void validate_tile_lists_kernel(const int32_t* __restrict__ offsets,
                                                                  const int32_t* __restrict__ cand, int num_tiles,
                                                                  int num_cand, int capacity, int num_prims,
                                                                  int32_t* __restrict__ status) {
  const int64_t stride = (int64_t)blockDim.x * gridDim.x;
  const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t tile = first; tile < num_tiles; tile += stride) {
    const int start = offsets[tile];
    const int end = offsets[tile + 1];
    if (start < 0 || end < start || end > num_cand || (tile == 0 && start != 0) ||
        (tile == num_tiles - 1 && end != num_cand)) {
      atomicOr(status, 1);
      continue;
    }
    const int count = end - start;
    if (capacity > 0 && count > capacity) {
      atomicOr(status, 2);
      atomicMax(status + 1, count);
    }
  }
  bool invalid = false;
  for (int64_t i = first; i < num_cand; i += stride) {
    const int p = cand[i];
    invalid |= (p < 0) || (p >= num_prims);
  }
  if (invalid) atomicOr(status, 4);
}

// d / max(|d|, 1e-12) per ray, as torch.nn.functional.normalize(ray_d, dim=-1) rounds it on this device
// (scannet/cumodel.py:1088): the squares are summed as (x^2 + z^2) + y^2 -- the order of torch's reduction over a
// last dimension of three -- then an exactly rounded square root and three exactly rounded divisions.  One launch
// in place of the library's four.
__global__ __launch_bounds__(256) void normalize_rays_kernel(const float* __restrict__ d, long long n,
                                                             float* __restrict__ out) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const Float3 v = load3(d, i);
  float ux, uy, uz;
  unit_direction(v.x, v.y, v.z, ux, uy, uz);
  store3(out, i, ux, uy, uz);
}

// The per-frame preparations that depend on nothing but the rays (and the scene), in one launch: blocks
// [0, ray_blocks) write the unit directions (normalize_rays_kernel's statements), the next tile_blocks blocks the
// tiles' ray pyramids for the sort (a wavefront per tile, from the directions as given: it does not wait for the unit
// vectors), the blocks after them the sort's frame records (if asked for).  (Blocks of the first two kinds taking
// turns instead: 20.1 us at 1200x680 against 14.6.)
__global__ __launch_bounds__(256) void frame_prologue_kernel(const float* __restrict__ d, long long n,
                                                             float* __restrict__ unit, int ray_blocks,
                                                             const float* __restrict__ rays_o, TileGeom g,
                                                             int tile_blocks, TilePyramidRec* __restrict__ pyramids,
                                                             const PrimRecord* __restrict__ prims, int N,
                                                             SortRec* __restrict__ frame) {
  const int b = (int)blockIdx.x;
  if (b < ray_blocks) {
    const long long i = (long long)b * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const Float3 v = load3(d, i);
    float ux, uy, uz;
    unit_direction(v.x, v.y, v.z, ux, uy, uz);
    store3(unit, i, ux, uy, uz);
  } else if (b < ray_blocks + tile_blocks) {
    const int tile = (b - ray_blocks) * (int)(blockDim.x >> 6) + (int)(threadIdx.x >> 6);
    if (tile < g.ntx * g.nty) write_tile_pyramid(rays_o, d, g, tile, pyramids);
  } else {
    write_frame_sort_record(rays_o, prims, N, frame,
                            (b - ray_blocks - tile_blocks) * (int)blockDim.x + (int)threadIdx.x);
  }
}

// One 256-thread workgroup per tile (mlpsp_sort_tile.hpp); super-blocks of tiles per XCD: the geometry records a
// tile gathers are mostly those of its neighbours.
// PYR: the tiles' ray pyramids come from records (the frame prologue's) instead of being built here.
// Tile t's list is cand[offsets[t] .. ends[t]) (ends = offsets + 1 for lists that follow one another without gaps).
// ASC: the ids of every list ascend (sort_one_tile_from).
template <bool PYR, bool ASC = false>
__global__ __launch_bounds__(kSortThreads) void sort_tiles_kernel(
    const float* __restrict__ rays_o, const float* __restrict__ rays_d, const PrimRecord* __restrict__ prims,
    const SortRec* __restrict__ frame, const TilePyramidRec* __restrict__ pyramids, const int32_t* __restrict__ cand,
    const int32_t* __restrict__ offsets, const int32_t* __restrict__ ends, TileGeom g, int family, int capacity,
    float cull_r2, int num_prims, int32_t* __restrict__ sorted_ids, float* __restrict__ sorted_keys) {
  const int tile = superblock_tile(blockIdx.x, g.ntx, g.nty);
  if (tile < 0) return;
  const int start = offsets[tile], len = ends[tile] - start;
  if (len <= 64 && len <= capacity) {       // a short list: the first wavefront alone, in registers
    if (len > 0 && threadIdx.x < 64)
      sort_small_tile<PYR>(rays_o, rays_d, prims, frame, pyramids, cand, g, family, cull_r2, num_prims, sorted_ids, sorted_keys,
                      tile, start, len);
    return;
  }
  __shared__ SortLds<MLPSP_TILE_CAPACITY_MAX> lds;
  sort_one_tile<MLPSP_TILE_CAPACITY_MAX, PYR, ASC>(lds, rays_o, rays_d, prims, frame, pyramids, cand, offsets, ends, g, family, capacity,
                                         cull_r2, num_prims, sorted_ids, sorted_keys, tile);
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_version(void) { return MLPSP_VERSION; }

MLPSP_API const char* mlpsp_strerror(int code) {
  switch (code) {
    case MLPSP_OK: return "ok";
    case MLPSP_E_OFFSETS:
      return "tile_offsets must start at zero, end at the candidate-list length, and be monotonic/in bounds";
    case MLPSP_E_CAPACITY:
      return "tile candidate capacity exceeded; refusing to truncate or use an inconsistent forward/backward order";
    case MLPSP_E_IDS: return "candidate primitive IDs must be in [0, num_primitives)";
    case MLPSP_E_PIXEL_OVERFLOW:
      return "per-pixel intersection capacity 256 exceeded; refusing to return a silently truncated result";
    case MLPSP_E_NONFINITE: return "non-finite operand or activation in the reduced-precision MLP";
    case MLPSP_E_ARGUMENT: return "invalid argument";
    case MLPSP_E_RUNTIME: return "HIP runtime error";
    case MLPSP_E_SCRATCH: return "scratch buffer too small for this input";
    case MLPSP_E_MIXED_ORIGINS: return "Each tile must use a single camera origin";
    case MLPSP_E_WIDE_CONE: return "Tile ray cone spans >=90 degrees";
    default: return "unknown mlpsp status";
  }
}

MLPSP_API int mlpsp_normalize_rays(const float* rays_d_dev, long long num_rays, float* unit_dirs_dev,
                                   mlpsp_stream_t stream) {
  if (num_rays < 0) return MLPSP_E_ARGUMENT;
  if (num_rays == 0) return MLPSP_OK;
  if (!rays_d_dev || !unit_dirs_dev) return MLPSP_E_ARGUMENT;
  if (num_rays > 2147483647LL * 256) return MLPSP_E_ARGUMENT;
  hipLaunchKernelGGL(normalize_rays_kernel, dim3((unsigned)((num_rays + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     rays_d_dev, num_rays, unit_dirs_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API size_t mlpsp_tile_pyramids_bytes(int width, int height, int tile_w, int tile_h) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  return T <= 0 ? 0 : (size_t)T * sizeof(TilePyramidRec);
}

MLPSP_API int mlpsp_frame_prologue(const float* rays_d_dev, float* unit_dirs_dev, const float* rays_o_dev, int width,
                                   int height, int tile_w, int tile_h, void* tile_pyramids_dev,
                                   const void* prim_records_dev, int num_primitives, void* frame_records_dev,
                                   mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0 || T > 2147483647LL) return MLPSP_E_ARGUMENT;
  const long long num_rays = (long long)width * height;
  if (!rays_d_dev || !unit_dirs_dev) return MLPSP_E_ARGUMENT;
  if (tile_pyramids_dev && (!rays_o_dev || reinterpret_cast<uintptr_t>(tile_pyramids_dev) % 32 != 0)) return MLPSP_E_ARGUMENT;
  if (frame_records_dev &&
      (!rays_o_dev || !prim_records_dev || num_primitives <= 0 || reinterpret_cast<uintptr_t>(frame_records_dev) % 64 != 0 ||
       reinterpret_cast<uintptr_t>(prim_records_dev) % 128 != 0))
    return MLPSP_E_ARGUMENT;
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  const long long ray_blocks = (num_rays + 255) / 256;
  const long long tile_blocks = tile_pyramids_dev ? (T + 3) / 4 : 0;
  const long long blocks = ray_blocks + tile_blocks + (frame_records_dev ? ceil_div(num_primitives, 256) : 0);
  if (blocks > 2147483647LL) return MLPSP_E_ARGUMENT;
  hipLaunchKernelGGL(frame_prologue_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, rays_d_dev, num_rays,
                     unit_dirs_dev, (int)ray_blocks, rays_o_dev, g, (int)tile_blocks, (TilePyramidRec*)tile_pyramids_dev,
                     (const PrimRecord*)prim_records_dev, num_primitives, (SortRec*)frame_records_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_prepare_primitives(const float* positions_dev, const float* log_scales_dev,
                                       const float* quats_dev, int num_primitives, void* prim_records_dev,
                                       mlpsp_stream_t stream) {
  if (num_primitives < 0) return MLPSP_E_ARGUMENT;
  if (num_primitives == 0) return MLPSP_OK;
  if (!positions_dev || !log_scales_dev || !quats_dev || !prim_records_dev) return MLPSP_E_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(prim_records_dev) % 128 != 0) return MLPSP_E_ARGUMENT;
  hipLaunchKernelGGL(prepare_primitives_kernel, dim3(ceil_div(num_primitives, 256)), dim3(256), 0,
                     (hipStream_t)stream, positions_dev, log_scales_dev, quats_dev, num_primitives,
                     (PrimRecord*)prim_records_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_validate_tile_lists(const int32_t* tile_offsets_dev, const int32_t* candidates_dev,
                                        int num_tiles, int num_candidates, int capacity, int num_primitives,
                                        int32_t* status_dev, int32_t status_host[2], mlpsp_stream_t stream) {
  if (num_tiles <= 0 || num_candidates < 0 || num_primitives < 0 || !tile_offsets_dev || !status_dev || !status_host)
    return MLPSP_E_ARGUMENT;
  if (num_candidates > 0 && !candidates_dev) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  MLPSP_HIP_TRY(hipMemsetAsync(status_dev, 0, 2 * sizeof(int32_t), s));
  const int64_t work = num_tiles > num_candidates ? num_tiles : num_candidates;
  int64_t blocks = (work + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(validate_tile_lists_kernel, dim3((unsigned)blocks), dim3(256), 0, s, tile_offsets_dev,
                     candidates_dev, num_tiles, num_candidates, capacity, num_primitives, status_dev);
  MLPSP_LAUNCH_CHECK();
  MLPSP_HIP_TRY(hipMemcpyAsync(status_host, status_dev, 2 * sizeof(int32_t), hipMemcpyDeviceToHost, s));
  MLPSP_HIP_TRY(hipStreamSynchronize(s));
  int mask = status_host[0] & (MLPSP_E_OFFSETS | MLPSP_E_CAPACITY | MLPSP_E_IDS);
  if (capacity <= 0) mask &= ~MLPSP_E_CAPACITY;
  return mask;
}

MLPSP_API size_t mlpsp_sort_frame_records_bytes(int num_primitives) {
  return num_primitives < 0 ? 0 : ((size_t)num_primitives + 1) * sizeof(SortRec);
}

MLPSP_API int mlpsp_sort_tiles(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                               int num_primitives, const int32_t* candidates_dev, const int32_t* tile_offsets_dev,
                               int width, int height, int tile_w, int tile_h, int key_family, int capacity,
                               float cull_threshold, void* frame_records_dev, int frame_records_ready,
                               const void* tile_pyramids_dev, const int32_t* tile_ends_dev, int ids_ascend,
                               int32_t* sorted_ids_dev, float* sorted_keys_dev, mlpsp_stream_t stream) {
  const int64_t T = checked_num_tiles(width, height, tile_w, tile_h);
  if (T <= 0 || T > 2147483647LL) return MLPSP_E_ARGUMENT;
  if (key_family != MLPSP_KEY_TSTAR && key_family != MLPSP_KEY_DEPTH) return MLPSP_E_ARGUMENT;
  if (capacity < 0 || capacity > MLPSP_TILE_CAPACITY_MAX) return MLPSP_E_ARGUMENT;
  if (capacity == 0) capacity = MLPSP_TILE_CAPACITY_MAX;
  if (!rays_o_dev || !rays_d_dev || !tile_offsets_dev || !candidates_dev || !sorted_ids_dev) return MLPSP_E_ARGUMENT;
  if (num_primitives <= 0 || !prim_records_dev) return MLPSP_E_ARGUMENT;
  if (sorted_ids_dev == candidates_dev) return MLPSP_E_ARGUMENT;   // not an in-place sort
  if (reinterpret_cast<uintptr_t>(frame_records_dev) % 64 != 0) return MLPSP_E_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(tile_pyramids_dev) % 32 != 0) return MLPSP_E_ARGUMENT;
  TileGeom g{width, height, tile_w, tile_h, ceil_div(width, tile_w), ceil_div(height, tile_h)};
  const int32_t* ends = tile_ends_dev ? tile_ends_dev : tile_offsets_dev + 1;
  // squared radius of the threshold ellipsoid in units of the scales, with a 2 % margin on the radius
  float cull_r2 = 0.f;
  if (cull_threshold > 0.f && cull_threshold < 1.f) cull_r2 = -2.0f * logf(cull_threshold) * 1.0404f + 1e-6f;
  // per-frame records for the origin of ray 0: every tile whose centre ray starts there takes its keys from them
  if (frame_records_dev && !frame_records_ready) {
    hipLaunchKernelGGL(frame_sort_records_kernel, dim3(ceil_div(num_primitives, 256)), dim3(256), 0, (hipStream_t)stream,
                       rays_o_dev, (const PrimRecord*)prim_records_dev, num_primitives, (SortRec*)frame_records_dev);
    MLPSP_LAUNCH_CHECK();
  }
  if (tile_pyramids_dev && ids_ascend)
    hipLaunchKernelGGL((sort_tiles_kernel<true, true>), dim3(superblock_grid(g.ntx, g.nty)), dim3(kSortThreads), 0,
                       (hipStream_t)stream, rays_o_dev, rays_d_dev, (const PrimRecord*)prim_records_dev,
                       (const SortRec*)frame_records_dev, (const TilePyramidRec*)tile_pyramids_dev, candidates_dev,
                       tile_offsets_dev, ends, g, key_family, capacity, cull_r2, num_primitives, sorted_ids_dev,
                       sorted_keys_dev);
  else if (tile_pyramids_dev)
    hipLaunchKernelGGL(sort_tiles_kernel<true>, dim3(superblock_grid(g.ntx, g.nty)), dim3(kSortThreads), 0,
                       (hipStream_t)stream, rays_o_dev, rays_d_dev, (const PrimRecord*)prim_records_dev,
                       (const SortRec*)frame_records_dev, (const TilePyramidRec*)tile_pyramids_dev, candidates_dev,
                       tile_offsets_dev, ends, g, key_family, capacity, cull_r2, num_primitives, sorted_ids_dev,
                       sorted_keys_dev);
  else
    hipLaunchKernelGGL(sort_tiles_kernel<false>, dim3(superblock_grid(g.ntx, g.nty)), dim3(kSortThreads), 0,
                       (hipStream_t)stream, rays_o_dev, rays_d_dev, (const PrimRecord*)prim_records_dev,
                       (const SortRec*)frame_records_dev, (const TilePyramidRec*)nullptr, candidates_dev,
                       tile_offsets_dev, ends, g, key_family, capacity, cull_r2, num_primitives, sorted_ids_dev,
                       sorted_keys_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
