// Hit records: what a render kernel hands to the feature-image kernels.
//
// The feature image is linear in the per-primitive attributes, so the render kernel only has to say, per
// work item (one wavefront = 64 pixels of a tile), WHICH primitives hit at least one of its pixels, in
// compositing order, and with which per-pixel coefficients.  An item cannot know in advance how many of
// its candidates will hit before its pixels saturate (at the 200k-primitive benchmark scene: 8 % of
// them), so records live in a pool that wavefronts draw from in chunks of 16 records with one atomic
// add per chunk; chunk_table maps (item, record number / 16) to the chunk.  An exhausted pool raises
// the overflow word and the item stops emitting; the host then repeats the frame with the worst-case
// pool (one record per candidate + 15 per item), which cannot overflow.
//
// Workspace layout (every part 256-byte aligned):
//   counters   int32[64]     [0] next free chunk, [1] overflow flag          (zeroed by the entry point)
//   item_hits  int32[items]  records emitted by each item
//   chunk_table int32[wpt * (P/16 + T + 1)]   index (w * stride) + (list_start >> 4) + tile + (m >> 4)
//   hit_ids    int32[pool_chunks * 16]
//   records    pool_chunks * 16 * record_bytes
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlpsp {

constexpr int kHitChunk = 16;
constexpr int kHitGrab = 4;      // chunks a wavefront draws from the pool per atomic

struct HitPool {
  int32_t* counters;
  int32_t* item_hits;
  int32_t* chunk_table;
  int32_t* hit_ids;
  unsigned char* records;
  int table_stride;   // P/16 + T + 1
  int pool_chunks;
  int record_bytes;
};

inline size_t hitpool_align(size_t v) { return (v + 255) & ~(size_t)255; }

// Bytes of a workspace for `pool_records` records (rounded up to whole chunks).
inline size_t hitpool_bytes(int64_t num_pairs, int64_t num_tiles, int waves_per_tile, int64_t pool_records,
                            int record_bytes) {
  const size_t chunks = (size_t)((pool_records + kHitChunk - 1) / kHitChunk);
  const size_t stride = (size_t)(num_pairs / kHitChunk + num_tiles + 1);
  return hitpool_align(64 * 4) + hitpool_align((size_t)num_tiles * waves_per_tile * 4) +
         hitpool_align(stride * waves_per_tile * 4) + hitpool_align(chunks * kHitChunk * 4) +
         hitpool_align(chunks * kHitChunk * (size_t)record_bytes) + 1536;   // slack: hitpool_carve keeps 1 KiB back
}

// Largest pool that fits in `bytes` -> HitPool (pool_chunks may be 0: every emission overflows).
inline HitPool hitpool_carve(void* workspace, size_t bytes, int64_t num_pairs, int64_t num_tiles, int waves_per_tile,
                             int record_bytes) {
  HitPool hp{};
  unsigned char* p = (unsigned char*)workspace;
  const size_t stride = (size_t)(num_pairs / kHitChunk + num_tiles + 1);
  hp.counters = (int32_t*)p;
  p += hitpool_align(64 * 4);
  hp.item_hits = (int32_t*)p;
  p += hitpool_align((size_t)num_tiles * waves_per_tile * 4);
  hp.chunk_table = (int32_t*)p;
  p += hitpool_align(stride * waves_per_tile * 4);
  const size_t used = (size_t)(p - (unsigned char*)workspace);
  hp.table_stride = (int)stride;
  hp.record_bytes = record_bytes;
  size_t chunks = 0;
  if (bytes > used + 1024) {
    // chunks * 16 * (4 + record_bytes) + alignment slack
    chunks = (bytes - used - 1024) / ((size_t)kHitChunk * (4 + (size_t)record_bytes));
    if (chunks > 0x7fffffffull / kHitChunk) chunks = 0x7fffffffull / kHitChunk;
  }
  hp.pool_chunks = (int)chunks;
  hp.hit_ids = (int32_t*)p;
  p += hitpool_align(chunks * kHitChunk * 4);
  hp.records = p;
  return hp;
}

// Smallest workspace a call accepts (tables, no pool).
inline size_t hitpool_min_bytes(int64_t num_pairs, int64_t num_tiles, int waves_per_tile) {
  return hitpool_bytes(num_pairs, num_tiles, waves_per_tile, 0, 0);
}

#if defined(__HIPCC__)
// Wave-uniform emitter state of one work item.
struct HitEmitter {
  int table_base;   // (w * stride) + (list_start >> 4) + tile
  int count;        // records emitted so far
  int chunk;        // current chunk, -1 once the pool is exhausted
};

__device__ __forceinline__ HitEmitter hit_emitter_begin(const HitPool& hp, int wave_slot, int list_start, int tile) {
  return HitEmitter{wave_slot * hp.table_stride + (list_start >> 4) + tile, 0, 0};
}

// Slot (record index in the pool) for the item's next record, or -1 on overflow.  Call with the whole
// wavefront active; the result is wave-uniform.  The pool is drawn kHitGrab chunks at a time (one atomic per 64
// records: the wavefront waits for its result, and every vector-memory wait behind it waits with it), the chunk
// table still has one entry per chunk.
__device__ __forceinline__ int hit_emitter_next(const HitPool& hp, HitEmitter& em, int lane) {
  if (em.chunk < 0) return -1;
  constexpr int kGroup = kHitChunk * kHitGrab;
  if ((em.count & (kGroup - 1)) == 0) {
    int c = 0;
    if (lane == 0) c = atomicAdd(hp.counters, kHitGrab);
    c = __builtin_amdgcn_readfirstlane(c);
    if (c + kHitGrab > hp.pool_chunks) {
      if (lane == 0) atomicExch(hp.counters + 1, 1);
      em.chunk = -1;
      return -1;
    }
    em.chunk = c;                       // first chunk of the group
  }
  const int within = em.count & (kGroup - 1);
  if ((within & (kHitChunk - 1)) == 0 && lane == 0)
    hp.chunk_table[em.table_base + (em.count >> 4)] = em.chunk + (within >> 4);
  const int slot = em.chunk * kHitChunk + within;
  ++em.count;
  return slot;
}

// Reader side: pool slot of record m of an item.
__device__ __forceinline__ int hit_slot(const HitPool& hp, int table_base, int m) {
  return hp.chunk_table[table_base + (m >> 4)] * kHitChunk + (m & (kHitChunk - 1));
}
#endif

}  // namespace mlpsp
