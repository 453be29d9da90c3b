// Host-side helpers shared by the translation units of libmlpsp_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/mlpsp.h"

#define MLPSP_API extern "C" __attribute__((visibility("default")))

// A failed HIP call maps to MLPSP_E_RUNTIME; the sticky error is cleared so that the caller's
// context stays usable (the reference's tests synchronise after every rejected call).
#define MLPSP_HIP_TRY(expr)                  \
  do {                                       \
    hipError_t e__ = (expr);                 \
    if (e__ != hipSuccess) {                 \
      (void)hipGetLastError();               \
      return MLPSP_E_RUNTIME;                \
    }                                        \
  } while (0)

#define MLPSP_LAUNCH_CHECK() MLPSP_HIP_TRY(hipGetLastError())

namespace mlpsp {

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// tiles_x * tiles_y with the overflow checks of np_tile_kernels.cu:4542-4551; 0 if unusable.
inline int64_t checked_num_tiles(int64_t W, int64_t H, int64_t TW, int64_t TH) {
  if (W <= 0 || H <= 0 || TW <= 0 || TH <= 0) return 0;
  const int64_t tx = 1 + (W - 1) / TW, ty = 1 + (H - 1) / TH;
  if (tx > 2147483647LL || ty > 2147483647LL || tx > 2147483647LL / ty) return 0;
  return tx * ty;
}

// The chip hands consecutive workgroup ids to its 8 XCDs in turn, and each XCD has its own L2.
// Kernels that want neighbouring work items to share an L2 launch 8*per_xcd workgroups and map
// blockIdx.x -> (blockIdx.x % 8) * per_xcd + blockIdx.x / 8, so XCD k owns the contiguous range
// [k*per_xcd, (k+1)*per_xcd) of logical work items.
constexpr int kNumXcd = 8;

// Tile kernels whose neighbouring tiles share most of their primitives use a two-dimensional version of the same
// idea: the tile grid is cut into super-blocks of kSuperSide x kSuperSide tiles and the super-blocks are dealt to
// the XCDs in turn, so the (up to) 64 tiles of a super-block run on one L2 while every XCD still gets an equal
// share of every image region.  Workgroup b belongs to XCD b % 8; it is that XCD's j-th workgroup, j = b / 8, and
// takes tile j % 64 of the XCD's (j / 64)-th super-block.  Tiles outside the image return -1.
constexpr int kSuperSide = 8;

inline unsigned superblock_grid(int ntx, int nty) {
  const int nsb = ((ntx + kSuperSide - 1) / kSuperSide) * ((nty + kSuperSide - 1) / kSuperSide);
  return (unsigned)(((nsb + kNumXcd - 1) / kNumXcd) * kNumXcd * kSuperSide * kSuperSide);
}

// j-th tile slot of XCD xcd
__device__ __forceinline__ int superblock_tile_of(int xcd, int j, int ntx, int nty) {
  constexpr int SB = kSuperSide;
  const int nsx = (ntx + SB - 1) / SB, nsy = (nty + SB - 1) / SB;
  const int sb = kNumXcd * (j / (SB * SB)) + xcd, within = j % (SB * SB);
  if (sb >= nsx * nsy) return -1;
  const int stx = (sb % nsx) * SB + within % SB, sty = (sb / nsx) * SB + within / SB;
  return (stx < ntx && sty < nty) ? sty * ntx + stx : -1;
}

__device__ __forceinline__ int superblock_tile(unsigned block, int ntx, int nty) {
  constexpr int SB = kSuperSide;
  const int nsx = (ntx + SB - 1) / SB, nsy = (nty + SB - 1) / SB;
  const int xcd = block % kNumXcd, j = block / kNumXcd;
  const int sb = kNumXcd * (j / (SB * SB)) + xcd, within = j % (SB * SB);
  if (sb >= nsx * nsy) return -1;
  const int stx = (sb % nsx) * SB + within % SB, sty = (sb / nsx) * SB + within / SB;
  return (stx < ntx && sty < nty) ? sty * ntx + stx : -1;
}

}  // namespace mlpsp
