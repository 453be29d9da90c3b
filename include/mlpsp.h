/* libmlpsp_hip: MI355X (gfx950) tile-based forward renderer for MLP Splatting -- C ABI.
 *
 * Every pointer named *_dev or documented as "device" is HIP device memory owned by the caller;
 * the library never allocates, frees or keeps device memory and never synchronises, except where
 * a function says it blocks.  All kernels are enqueued on `stream` (a hipStream_t passed as
 * void*; NULL = the default stream).  Functions return 0 (MLPSP_OK) or a bit mask of the MLPSP_E_*
 * values below; mlpsp_strerror() gives the message the reference raises for that condition.
 *
 * Tensor layouts are those of the reference extension (row-major, contiguous, f32 unless noted):
 *   rays_o, rays_d [B,3] (rays_d unit length), B = width*height, pixel = y*width + x
 *   positions, log_scales [N,3]; quats [N,4] unit (w,x,y,z)
 *   tile list: tile_offsets [T+1] int32, candidates [P] int32, tile = ty*ceil(width/tile_w) + tx
 *   freq, att [F]; W1 [N,H,12F] b1 [N,H] W2 [N,H,H] b2 [N,H] W3 [N,4,H] b3 [N,4]
 *   feat_attr [N,C] (slots = 1) or [N,slots,C] with slots in {4,5}, C <= 512
 *   outputs rgb [B,3], alpha [B,1], t [B,1], feat [B,C]
 *
 * Reference interface replaced: the pybind11 module of scannet/cuda/np_tile_kernels.cu:7224-7252
 * (forward entry points) and the PyTorch culling of scannet/cumodel.py:994-1070.
 */
#ifndef MLPSP_H
#define MLPSP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLPSP_OK 0
#define MLPSP_E_OFFSETS 1        /* tile_offsets not monotone / not covering the list (np_tile_kernels.cu:4499-4503) */
#define MLPSP_E_CAPACITY 2       /* a tile holds more candidates than the capacity (np_tile_kernels.cu:4506-4509) */
#define MLPSP_E_IDS 4            /* a candidate id is outside [0, N) (np_tile_kernels.cu:4513-4519) */
#define MLPSP_E_PIXEL_OVERFLOW 8 /* a pixel met a 257th hit in per-pixel order (np_tile_kernels.cu:798-809) */
#define MLPSP_E_NONFINITE 16     /* non-finite operand or activation in the bf16 MFMA path (rgb_wmma.cuh:260) */
#define MLPSP_E_ARGUMENT 32      /* a size or pointer argument is unusable */
#define MLPSP_E_RUNTIME 64       /* a HIP call failed */
#define MLPSP_E_SCRATCH 128      /* the scratch buffer is too small for this input: retry with a larger one */
#define MLPSP_E_MIXED_ORIGINS 256 /* ray-cone binning: a tile's rays do not share one origin (camera.py:121-122) */
#define MLPSP_E_WIDE_CONE 512    /* ray-cone binning: a tile's ray cone spans >= 90 degrees (camera.py:126) */

#define MLPSP_TILE_CAPACITY_MAX 2048 /* largest per-tile list the in-LDS sort accepts */
#define MLPSP_PIXEL_HIT_CAPACITY 256 /* per-pixel-order hit buffer (np_tile_kernels.cu:760) */
#define MLPSP_PRIM_RECORD_BYTES 128  /* bytes per primitive of the prepared geometry buffer */
#define MLPSP_MFMA_PACK_BYTES 7808   /* bytes per primitive of the packed matrix-core weight buffer */
#define MLPSP_SORT_RECORD_BYTES 64   /* bytes per primitive (+ one header slot) of the sort's per-frame records */
#define MLPSP_TILE_PYRAMID_BYTES 160 /* bytes per tile of the sort's ray-pyramid records */
#define MLPSP_BIN_STATIC_SCRATCH_BYTES 67108864 /* scratch array of mlpsp_bin_legacy_async_noalloc (64 MiB) */
#define MLPSP_BIN_STATIC_MAX_VIEWS 8           /* most views mlpsp_bin_legacy_async_noalloc accepts */

#define MLPSP_KEY_LIST_ORDER 0 /* consume the list as given (presorted kernel, np_tile_kernels.cu:4242-4478) */
#define MLPSP_KEY_TSTAR 1      /* Mahalanobis t* of the tile-centre ray (np_tile_kernels.cu:483-518) */
#define MLPSP_KEY_DEPTH 2      /* plain centre-ray depth (np_tile_kernels.cu:5538-5542) */

typedef void* mlpsp_stream_t;

/* Library version (major*10000 + minor*100 + patch).  MLPSP_VERSION is the version this header describes: a caller
 * built against it must find mlpsp_version() == MLPSP_VERSION (argument lists and the PrimRecord layout are not
 * compatible across versions). */
#define MLPSP_VERSION 303
int mlpsp_version(void);

/* Message for one MLPSP_E_* bit, worded as the reference's TORCH_CHECK for that condition
 * (np_tile_kernels.cu:4578-4598). */
const char* mlpsp_strerror(int code);

/* Per-primitive geometry in kernel-ready form: centre, exp(-2 log_s), unit quaternion, log_s, exp(2 log_s)
 * and the quaternion's rotation matrix (quats_dev must hold unit quaternions).
 * Replaces the per-candidate gathers + __expf of np_tile_kernels.cu:1947-1956, 676-678.
 * prim_records_dev: N * MLPSP_PRIM_RECORD_BYTES bytes, 128-byte aligned. */
int mlpsp_prepare_primitives(const float* positions_dev, const float* log_scales_dev, const float* quats_dev,
                             int num_primitives, void* prim_records_dev, mlpsp_stream_t stream);

/* Unit ray directions: unit_dirs[i] = rays_d[i] / max(|rays_d[i]|, 1e-12), bit for bit what
 * torch.nn.functional.normalize(ray_d, dim=-1) returns on this device (scannet/cumodel.py:1088, 1325, 1498), in one
 * launch.  rays_d_dev, unit_dirs_dev: num_rays x 3 floats, contiguous; they may be the same buffer. */
int mlpsp_normalize_rays(const float* rays_d_dev, long long num_rays, float* unit_dirs_dev, mlpsp_stream_t stream);

/* Tile-list validation = validate_tile_candidate_capacity (np_tile_kernels.cu:4485-4589).
 * capacity 0 = no cap (per-pixel and presorted entry points).  status_dev: 2 int32 of device
 * scratch.  BLOCKS: one 8-byte device-to-host copy, then returns the status mask;
 * status_host[0] = mask, status_host[1] = largest over-capacity tile length. */
int mlpsp_validate_tile_lists(const int32_t* tile_offsets_dev, const int32_t* candidates_dev, int num_tiles,
                              int num_candidates, int capacity, int num_primitives, int32_t* status_dev,
                              int32_t status_host[2], mlpsp_stream_t stream);

/* Legacy screen-space culling, sparse: replaces the dense [tiles x primitives] overlap matrix of
 * scannet/cumodel.py:994-1070 (one camera) and :838-949 (tile_view_ids_dev != NULL: K views, tile
 * t uses view tile_view_ids_dev[t]).  view_matrices: K row-major 4x4 on the HOST, proj: 4x4 on
 * the host.  Within a tile, candidate ids ascend.
 * Step 1 (count): writes exclusive offsets to tile_offsets_dev[T+1] (16-byte aligned); BLOCKS to return the total
 *   in counts_out[0] and the length of the longest tile list in counts_out[1] (what the capacity
 *   check of the render entry points compares with MLPSP_MAX_TILE_PRIMS).  scratch_dev: at least mlpsp_bin_scratch_bytes() bytes, 256-byte aligned,
 *   reused by step 2; MLPSP_E_SCRATCH asks for a larger one (primitives spanning very many tiles).
 * Step 2 (fill): writes candidates_dev[num_pairs]. */
size_t mlpsp_bin_scratch_bytes(int num_primitives, int num_views, int width, int height, int tile);
int mlpsp_bin_legacy_count(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                           const float* view_matrices_host, int num_views, const int32_t* tile_view_ids_dev,
                           const float* proj_host, int width, int height, int tile, float threshold,
                           void* scratch_dev, size_t scratch_bytes, int32_t* tile_offsets_dev,
                           int64_t counts_out[2], mlpsp_stream_t stream);
/* The same lists without any host synchronisation, for callers that queue a whole frame: candidates_dev
 * holds cand_capacity entries chosen by the caller (e.g. last frame's count plus a margin).
 * counts_dev (device int64[4]) receives {pairs, longest tile list, level-1 scratch entries, guard}.  If the
 * pairs exceed cand_capacity or the level-1 lists overflow the scratch, guard = 1 and EVERY tile list is left
 * empty (offsets all zero, nothing written to candidates_dev), so that kernels already queued behind this
 * call touch nothing; the caller reads counts_dev when it next synchronises, enlarges what was too small
 * and repeats the frame.  No counterpart in the reference (its culling is synchronous PyTorch). */
int mlpsp_bin_legacy_async(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                           const float* view_matrices_host, int num_views, const int32_t* tile_view_ids_dev,
                           const float* proj_host, int width, int height, int tile, float threshold,
                           void* scratch_dev, size_t scratch_bytes, int32_t* tile_offsets_dev,
                           int32_t* candidates_dev, int64_t cand_capacity, int64_t* counts_dev,
                           mlpsp_stream_t stream);

/* mlpsp_bin_legacy_async for ONE view whose two matrices are device tensors (4x4 row-major float each), as the
 * reference's evaluators hold them (scannet/eval_rgb_psnr.py:465-466): nothing is copied to the host, so a frame
 * that starts with this call starts without a synchronisation.  Same lists and counts, bit for bit (the focal
 * length is formed on the device with the host's expression). */
int mlpsp_bin_legacy_async_device_matrices(const float* positions_dev, const float* log_scales_dev,
                                           int num_primitives, const float* view_matrix_dev, const float* proj_dev,
                                           int width, int height, int tile, float threshold, void* scratch_dev,
                                           size_t scratch_bytes, int32_t* tile_offsets_dev, int32_t* candidates_dev,
                                           int64_t cand_capacity, int64_t* counts_dev, mlpsp_stream_t stream);
/* The lists of mlpsp_bin_legacy_async_device_matrices in SEGMENTS, for a frame that is queued whole: tile t owns
 * candidates_dev[t * segment_stride .. (t + 1) * segment_stride) and its list -- the same ids in the same ascending
 * order -- is the first tile_ends_dev[t] - t * segment_stride entries of it; tile_offsets_dev[t] = t * segment_stride
 * (T + 1 entries), tile_ends_dev holds T entries, candidates_dev T * segment_stride.  The render path accepts at most
 * its tile capacity (1,536 by default) entries per tile anyway, so with segment_stride = that capacity nothing is
 * lost, and the binning needs neither a count of the candidates before it writes them nor a
 * buffer sized by an estimate: level 2 tests and writes in one launch (three launches in all instead of four, and
 * no candidate-capacity guard).  A tile with more than segment_stride candidates keeps the first segment_stride and
 * raises counts_dev[1] to its full length (counts_dev[1] is 0 when every tile fits): the caller reports the
 * capacity error of np_tile_kernels.cu:4578-4588 from it.  counts_dev = {0, that maximum, level-1 scratch entries,
 * guard}; guard = 1 (level-1 scratch too small) leaves every list empty, as in mlpsp_bin_legacy_async.
 * mlpsp_sort_tiles and mlpsp_render_tilecenter_mfma_feat take such lists through their tile_ends_dev argument.
 * No counterpart in the reference (its culling is synchronous PyTorch, scannet/cumodel.py:994-1070). */
int mlpsp_bin_segments_async_device_matrices(const float* positions_dev, const float* log_scales_dev,
                                             int num_primitives, const float* view_matrix_dev, const float* proj_dev,
                                             int width, int height, int tile, float threshold, void* scratch_dev,
                                             size_t scratch_bytes, int segment_stride, int32_t* tile_offsets_dev,
                                             int32_t* tile_ends_dev, int32_t* candidates_dev, int64_t* counts_dev,
                                             mlpsp_stream_t stream);
int mlpsp_bin_legacy_fill(int num_primitives, int num_views, const int32_t* tile_view_ids_dev, int width,
                          int height, int tile, const void* scratch_dev, size_t scratch_bytes,
                          const int32_t* tile_offsets_dev, int32_t* candidates_dev, mlpsp_stream_t stream);

/* mlpsp_bin_legacy_async without a scratch argument and without any allocation.  No counterpart in the reference;
 * it is for callers that cannot allocate device memory where they call the renderer: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch is a device array inside the library
 * (mlpsp_bin_static_scratch_bytes() = MLPSP_BIN_STATIC_SCRATCH_BYTES bytes, held on every GPU the library runs on
 * until the process ends); inputs whose mlpsp_bin_scratch_bytes() exceed it return MLPSP_E_SCRATCH, more than
 * MLPSP_BIN_STATIC_MAX_VIEWS views MLPSP_E_ARGUMENT (the matrices travel as kernel arguments).  Same outputs,
 * guard behaviour and launches as mlpsp_bin_legacy_async, except that the level-1 lists get all of the array that
 * the rest leaves free (their overflow -- counts_dev[3] = 1 with counts_dev[2] entries -- is therefore rarer than with
 * a scratch of mlpsp_bin_scratch_bytes(); if it still happens the input needs mlpsp_bin_legacy_async with a larger
 * scratch); nothing is cleared with a memset (a fill kernel where needed), so the call may be captured.  All calls on one GPU share the one array: calls that overlap on a GPU
 * (two streams, two threads) race and must be serialised by the caller. */
size_t mlpsp_bin_static_scratch_bytes(void);
int mlpsp_bin_legacy_async_noalloc(const float* positions_dev, const float* log_scales_dev, int num_primitives,
                                   const float* view_matrices_host, int num_views, const int32_t* tile_view_ids_dev,
                                   const float* proj_host, int width, int height, int tile, float threshold,
                                   int32_t* tile_offsets_dev, int32_t* candidates_dev, int64_t cand_capacity,
                                   int64_t* counts_dev, mlpsp_stream_t stream);

/* Ray-cone culling from the actual rays = ray_cone_candidates (scannet/camera.py:102-146), for
 * cameras that are not a centred pinhole.  Same two steps and blocking behaviour as the legacy
 * binning; tile <= 16.  Within a tile, candidate ids ascend. */
size_t mlpsp_bin_raycone_scratch_bytes(int num_primitives, int width, int height, int tile);
int mlpsp_bin_raycone_count(const float* rays_o_dev, const float* rays_d_dev, const float* positions_dev,
                            const float* log_scales_dev, int num_primitives, int width, int height, int tile,
                            float threshold, void* scratch_dev, size_t scratch_bytes, int32_t* tile_offsets_dev,
                            int64_t* num_pairs_out, mlpsp_stream_t stream);
int mlpsp_bin_raycone_fill(int num_primitives, int width, int height, int tile, const void* scratch_dev,
                           size_t scratch_bytes, const int32_t* tile_offsets_dev, int32_t* candidates_dev,
                           mlpsp_stream_t stream);

/* Per-tile depth-key sort = the in-kernel cub::BlockRadixSort of np_tile_kernels.cu:1929-1990,
 * materialised: sorted_ids_dev[P] holds, tile by tile, the candidates in ascending key order, ties
 * in list order; entries past min(len, capacity) keep list order.  sorted_keys_dev may be NULL.
 * capacity <= MLPSP_TILE_CAPACITY_MAX (0 = that maximum).
 * cull_threshold: 0 = off.  In (0,1) (the render's score threshold): a candidate that provably hits
 * no ray of its tile at that threshold is written as ~id (negative).  The render entry points skip
 * negative ids, so images are unchanged; ~ recovers the plain sorted list.  Has no counterpart in the
 * reference, whose kernels run the full ray test on every candidate.
 * prim_records_dev holds num_primitives records.  Null pointers (sorted_keys_dev aside) return MLPSP_E_ARGUMENT;
 * a candidate id outside [0, num_primitives) -- a list that was not validated -- is not dereferenced: it sorts
 * last with the invalid key and is passed on as it is (the render entry points skip such ids).
 * frame_records_dev: NULL, or mlpsp_sort_frame_records_bytes(num_primitives) bytes of scratch, 64-byte aligned.
 * With it, one more launch first writes a 64-byte record per primitive for the origin of ray 0 -- the rotated
 * offset centre - origin of the key (np_tile_kernels.cu:483-500), which depends on the primitive alone when the
 * rays share an origin -- and every tile whose centre ray starts at that origin takes its keys from those records
 * (one quaternion rotation per candidate instead of two; same expressions, same key bits); other tiles, and every
 * tile without the scratch, evaluate the key in full.  Sorted ids and keys do not depend on it.
 * frame_records_ready != 0: the records are there already -- mlpsp_frame_prologue wrote them, for these rays and
 * these primitive records, earlier on the same stream -- and no launch is added.
 * tile_pyramids_dev: NULL, or the mlpsp_tile_pyramids_bytes() bytes that mlpsp_frame_prologue wrote for these rays
 * and this tile size earlier on the same stream (32-byte aligned): the four side planes of every tile's rays, which
 * the culling tests candidates against.  Without them every wavefront of a tile builds the planes from the tile's
 * 64 rays itself.  Keys and order do not depend on it; the two builds of the planes differ in their last bits, so a
 * candidate on the very edge of the culling's margin may be struck by one and not the other (the images are the
 * same: nothing that hits is ever struck).
 * tile_ends_dev: NULL (tile t's list ends where tile t + 1's begins: tile_offsets_dev[t + 1]) or T ends of lists
 * that lie in segments (mlpsp_bin_segments_async_device_matrices); the sorted lists are written to the same places.
 * ids_ascend != 0: the caller vouches that the ids of every list ascend, as the mlpsp_bin_* entry points write them
 * (ties in list order are then ties in id order and the kernel sorts (key, id) words, which spares it a gather of the
 * ids at the end; used with tile_pyramids_dev, ignored without).  Lists in any other order must pass 0. */
size_t mlpsp_sort_frame_records_bytes(int num_primitives);
size_t mlpsp_tile_pyramids_bytes(int width, int height, int tile_w, int tile_h);
/* The per-frame preparations that need nothing but the rays (and the scene), in ONE launch: the unit directions of
 * mlpsp_normalize_rays for the width * height rays at rays_d_dev; with tile_pyramids_dev != NULL the sort's ray
 * pyramid of every tile (formed from the directions as given; needs rays_o_dev); with frame_records_dev != NULL the sort's frame records for the origin of ray 0 (needs rays_o_dev and
 * the primitive records).  No counterpart in the reference, which normalises with torch (scannet/cumodel.py:1088)
 * and runs the full ray test on every candidate. */
int mlpsp_frame_prologue(const float* rays_d_dev, float* unit_dirs_dev, const float* rays_o_dev, int width, int height,
                         int tile_w, int tile_h, void* tile_pyramids_dev, const void* prim_records_dev,
                         int num_primitives, void* frame_records_dev, mlpsp_stream_t stream);
int mlpsp_sort_tiles(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                     int num_primitives, const int32_t* candidates_dev, const int32_t* tile_offsets_dev, int width,
                     int height, int tile_w, int tile_h, int key_family, int capacity, float cull_threshold,
                     void* frame_records_dev, int frame_records_ready, const void* tile_pyramids_dev,
                     const int32_t* tile_ends_dev, int ids_ascend, int32_t* sorted_ids_dev, float* sorted_keys_dev,
                     mlpsp_stream_t stream);

/* Tile-centre-order forward, scalar f32 (render_tiles_kernel_tilecenter_order,
 * np_tile_kernels.cu:1837-2137; with out_t_dev != NULL also the expected depth of :5432-5719).
 * order_dev: the tile lists in processing order (mlpsp_sort_tiles output, or the candidates
 * themselves for MLPSP_KEY_LIST_ORDER).  counters_dev: NULL or 4 int64 {unused, tile-primitives
 * processed, tile-primitives with a hit, hits}, accumulated (zero them first).
 * Launches too small to fill the chip (at most 1,024 wavefronts; the 72-32-32-4 and 72-16-16-4 shapes) take a kernel
 * that requests the next list entry's operands ahead, and at most 512 without counters one that puts two wavefronts
 * on every 64 pixels; same bits.  MLPSP_F32_AHEAD=0/1/2 in the environment picks the form by hand, MLPSP_F32_SCALAR=1
 * the kernel without matrix instructions. */
int mlpsp_render_tilecenter_f32(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                const float* att_dev, int num_frequencies, const float* W1, const float* b1,
                                const float* W2, const float* b2, const float* W3, const float* b3,
                                int num_primitives, int hidden, int width, int height, int tile_w, int tile_h,
                                float threshold, float* out_rgb_dev, float* out_alpha_dev, float* out_t_dev,
                                int64_t* counters_dev, mlpsp_stream_t stream);

/* Pruning-statistics forward (render_tiles_kernel_tilecenter_order_stats, np_tile_kernels.cu:2139-2519,
 * wrapper :5349-5428): renders like mlpsp_render_tilecenter_f32 and, per processed primitive p, adds to
 * stat_sum_w[p] the sum over the tile's pixels of the compositing weight w, raises stat_max_w[p] to the
 * largest w, adds to stat_hits[p] the number of pixels with w > 1e-8, to stat_sum_werr[p] the sum of
 * w * err over pixels with w > 0.1 (err = L1 distance of the pixel's colour after this step from
 * gt_rgb_dev [B,3]) and to stat_contrib[p] their number.  The five buffers [N] are updated in place with
 * atomics (the last two may be NULL); the reference sorts this kernel's tiles with MLPSP_KEY_DEPTH. */
int mlpsp_render_tilecenter_stats_f32(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                      const int32_t* order_dev, const int32_t* tile_offsets_dev,
                                      const float* freq_dev, const float* att_dev, int num_frequencies,
                                      const float* W1, const float* b1, const float* W2, const float* b2,
                                      const float* W3, const float* b3, int num_primitives, int hidden, int width,
                                      int height, int tile_w, int tile_h, float threshold, const float* gt_rgb_dev,
                                      float* out_rgb_dev, float* out_alpha_dev, float* stat_sum_w_dev,
                                      float* stat_max_w_dev, int32_t* stat_hits_dev, float* stat_sum_werr_dev,
                                      int32_t* stat_contrib_dev, mlpsp_stream_t stream);

/* Training-records forward (render_tiles_training_records, np_tile_kernels.cu:6897-6998; kernel :2925-3206
 * in record modes 1 and 3).  t* order, f32, hidden <= 32.  Per pixel, one record per hit taken while the
 * pixel is live (T >= 1e-3) and holds fewer than max_hits records: ids [R], x6 [R,6] (ray direction, world
 * offset), masks [R,2] (ReLU bit masks of the two hidden layers), raw [R,8] (R, G, B, sigma_raw, T before the
 * hit, alpha, decay, sigma logit), gates [R,4]; rgb/alpha are the composite of the records.
 * Step 1 (count): counts_dev [B] int32.  The caller scans them into record_offsets_dev [B+1] int64
 * (exclusive) and allocates R = record_offsets[B] records.  Step 2 (emit) writes them.
 * overflow_dev (int32, zeroed by the count step): 1 if a live pixel reached max_hits -- the reference
 * raises "hit capacity" then (:4601-4609); nothing is truncated silently.
 * render_order: 0 = the record kernels' rounding of layer 2 (bias added after a sum started at zero,
 * np_tile_kernels.cu:349-353); 1 = the render kernels' (sum started at the bias): image, alpha and every record
 * field are then those of mlpsp_render_tilecenter_f32 bit for bit, so a differentiable render can use the
 * records forward AS its forward.  1 needs the 72->32->32->4 shape with 16-byte aligned weights. */
int mlpsp_records_count(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                        const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                        const float* att_dev, int num_frequencies, const float* W1, const float* b1, const float* W2,
                        const float* b2, const float* W3, const float* b3, int num_primitives, int hidden, int width,
                        int height, int tile_w, int tile_h, float threshold, int max_hits, int render_order,
                        int32_t* counts_dev, int32_t* overflow_dev, mlpsp_stream_t stream);
int mlpsp_records_emit(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                       const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                       const float* att_dev, int num_frequencies, const float* W1, const float* b1, const float* W2,
                       const float* b2, const float* W3, const float* b3, int num_primitives, int hidden, int width,
                       int height, int tile_w, int tile_h, float threshold, int max_hits, int render_order,
                       float gating_beta, float gating_temp, const int64_t* record_offsets_dev, int32_t* ids_dev, float* x6_dev,
                       int32_t* masks_dev, float* raw_dev, float* gates_dev, float* out_rgb_dev, float* out_alpha_dev,
                       int32_t* overflow_dev, mlpsp_stream_t stream);

/* Training-records forward with the MLP on the matrix cores = render_training_wmma_kernel
 * (scannet/cuda/training_wmma.cuh:62-253; wrapper render_tiles_training_records_wmma :267-357).  8x8 tiles,
 * 72->32->32->4 MLP with six frequencies; packed_dev = mlpsp_pack_mfma_weights of the six weight tensors in
 * the precision of use_bf16.  order_dev is the tile list sorted by mlpsp_sort_tiles (t* key): the reference
 * sorts inside its kernel, here the sorted list is shared with the scalar record forward.  Geometry, record
 * order, x6, decay and gates are the f32 expressions of mlpsp_records_count/emit; R, G, B, sigma, alpha follow
 * the reduced-precision MLP.  Same two steps and outputs as mlpsp_records_count/emit.  status_dev (int32, NOT
 * cleared here: the caller clears it once per frame) collects 1 = non-finite operand, activation or output
 * (the reference repeats the whole frame with the scalar f32 record forward), 2 = a live pixel reached
 * max_hits (hit capacity, refused), 4 = the emit step met a pixel whose hit count differs from its offsets
 * interval (nothing is written outside the interval). */
int mlpsp_records_mfma_count(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                             const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                             const float* att_dev, const void* packed_dev, int num_primitives, int width, int height,
                             float threshold, int max_hits, int use_bf16, int32_t* counts_dev, int32_t* status_dev,
                             mlpsp_stream_t stream);
int mlpsp_records_mfma_emit(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                            const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                            const float* att_dev, const void* packed_dev, int num_primitives, int width, int height,
                            float threshold, int max_hits, int use_bf16, float gating_beta, float gating_temp,
                            const int64_t* record_offsets_dev, int64_t total_records, int32_t* ids_dev, float* x6_dev,
                            int32_t* masks_dev, float* raw_dev, float* gates_dev, float* out_rgb_dev,
                            float* out_alpha_dev, int32_t* status_dev, mlpsp_stream_t stream);

/* flag_dev[0] = 1 if any element of the num_arrays (<= 16) f32 device arrays is NaN or infinite, else 0 =
 * training_wmma_finite_kernel (scannet/cuda/training_wmma.cuh:24-60): one fused read-only scan in front of the
 * reduced-precision record forward, which refuses non-finite inputs.  arrays_dev and lengths are HOST arrays of
 * device pointers and element counts; empty arrays are skipped. */
int mlpsp_all_finite(const float* const* arrays_dev, const int64_t* lengths, int num_arrays, int32_t* flag_dev,
                     mlpsp_stream_t stream);

/* Workspace of the feature renders below.  The render kernel hands the feature kernel one "hit record"
 * per (64-pixel wavefront of a tile, primitive that hits one of its pixels); how many there will be is
 * only known after the frame (early termination), so records come from a pool of pool_records records.
 * pool_records < 0 asks for the worst case (one per candidate and wavefront + 63 per wavefront), which can
 * never run out; a smaller pool that runs out sets the call's overflow status and the caller repeats the
 * frame with a larger one.  fp16_records: 0 for mlpsp_render_tilecenter_feat_f32, 1 for
 * mlpsp_render_tilecenter_mfma_feat (tile_w = tile_h = 8).  0 on bad arguments. */
size_t mlpsp_feat_workspace_bytes(int64_t num_pairs, int width, int height, int tile_w, int tile_h, int feat_slots,
                                  int fp16_records, int64_t pool_records);

/* Tile-centre-order forward with the gated feature channel, scalar f32
 * (render_tiles_kernel_tilecenter_order_with_feat, np_tile_kernels.cu:5794-6112).
 * feat_slots: 1 (feat_attr [N,C]), 4 or 5 ([N,slots,C]); feat_channels <= 512.
 * out_feat_dev [B,C] is fully written (no pre-zeroing needed).  num_pairs = length of order_dev.
 * workspace_dev: 256-byte aligned, at least mlpsp_feat_workspace_bytes(.., pool_records = 0) bytes
 * (MLPSP_E_SCRATCH otherwise); whatever it holds beyond that is the record pool.
 * status_dev[0] (device int32) = 1 if the pool ran out: out_feat_dev is then incomplete (RGB and alpha
 * are complete either way). */
int mlpsp_render_tilecenter_feat_f32(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                     const int32_t* order_dev, const int32_t* tile_offsets_dev,
                                     const float* freq_dev, const float* att_dev, int num_frequencies,
                                     const float* W1, const float* b1, const float* W2, const float* b2,
                                     const float* W3, const float* b3, int num_primitives, int hidden,
                                     const float* feat_attr_dev, int feat_slots, int feat_channels,
                                     float gating_beta, float gating_temp, int width, int height, int tile_w,
                                     int tile_h, float threshold, int64_t num_pairs, void* workspace_dev,
                                     size_t workspace_bytes, float* out_rgb_dev, float* out_alpha_dev,
                                     float* out_feat_dev, int32_t* status_dev, mlpsp_stream_t stream);

/* Per-pixel-order forward (render_tiles_kernel_with_sort[_and_feat], np_tile_kernels.cu:715-1208):
 * every pixel blends its own hits in order of its own t.  candidates_dev is the unsorted tile list.
 * out_feat_dev == NULL renders RGB only.  workspace_dev: mlpsp_per_pixel_workspace_bytes() bytes,
 * 256-byte aligned.  BLOCKS (one 4-byte readback): returns MLPSP_E_PIXEL_OVERFLOW if some pixel
 * met a 257th hit, in which case the outputs must be discarded. */
size_t mlpsp_per_pixel_workspace_bytes(int width, int height, int tile_w, int tile_h);
int mlpsp_render_per_pixel_f32(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                               const int32_t* candidates_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                               const float* att_dev, int num_frequencies, const float* W1, const float* b1,
                               const float* W2, const float* b2, const float* W3, const float* b3,
                               int num_primitives, int hidden, const float* feat_attr_dev, int feat_slots,
                               int feat_channels, float gating_beta, float gating_temp, int width, int height,
                               int tile_w, int tile_h, float threshold, void* workspace_dev, size_t workspace_bytes,
                               float* out_rgb_dev, float* out_alpha_dev, float* out_feat_dev, mlpsp_stream_t stream);

/* Training records in per-pixel order: the traversal of render_tiles_backward_count_per_pixel and
 * render_tiles_backward_emit_per_pixel (scannet/cuda/np_tile_kernels.cu:1211-1836, wrappers :6290-6400; called from
 * _TileRenderAutogradFn.backward mode 0, scannet/cumodel.py:297-331) with the record schema of mlpsp_records_emit:
 * every pixel's hits (at most 256; a 257th returns MLPSP_E_PIXEL_OVERFLOW) in the order of its own t, blended until
 * the transmittance falls below 1e-3.  count leaves the number of blended hits per pixel in counts_dev [W*H];
 * the caller scans them into record_offsets_dev [W*H+1] (int64) and calls emit, which writes ids [R], x6 [R,6],
 * masks [R,2], raw [R,8], gates [R,4] and the image (rgb [W*H,3], alpha [W*H]).  The reference's emit kernel also
 * composes the adjoints; here they come from mlpsp_records_reverse_adjoints over these records.  workspace as for
 * mlpsp_render_per_pixel_f32; blocking (one 4-byte read-back), like it.  hidden <= 32. */
int mlpsp_records_per_pixel_count(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* candidates_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, int width, int height, int tile_w, int tile_h, float threshold,
    void* workspace_dev, size_t workspace_bytes, int32_t* counts_dev, mlpsp_stream_t stream);
int mlpsp_records_per_pixel_emit(
    const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev, const int32_t* candidates_dev,
    const int32_t* tile_offsets_dev, const float* freq_dev, const float* att_dev, int num_frequencies,
    const float* W1, const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
    int num_primitives, int hidden, float gating_beta, float gating_temp, int width, int height, int tile_w,
    int tile_h, float threshold, void* workspace_dev, size_t workspace_bytes, const int64_t* record_offsets_dev,
    int64_t total_records, int32_t* ids_dev, float* x6_dev, int32_t* masks_dev, float* raw_dev, float* gates_dev,
    float* out_rgb_dev, float* out_alpha_dev, mlpsp_stream_t stream);

/* Matrix-core path for the released 72->32->32->4 MLP (F = 6, H = 32), 8x8 tiles; the counterpart of
 * render_tiles_rgb_wmma (scannet/cuda/rgb_wmma.cuh:75-274).
 * mlpsp_pack_mfma_weights: rounds W1, W2, W3 to bf16 (use_bf16 != 0) or fp16 and stores them, with the
 *   f32 biases, in MFMA operand order: mlpsp_mfma_pack_bytes(N) bytes, 128-byte aligned.  Done once per
 *   set of weights (the reference re-casts them for every tile and primitive, rgb_wmma.cuh:162-174).
 * mlpsp_render_tilecenter_mfma: geometry, activations and compositing in f32; encoded inputs, weights
 *   and hidden activations in bf16/fp16 with f32 accumulation.  status_dev: 16 int32 of device
 *   scratch, zeroed by the call; status_dev[0] becomes 1 if a non-finite operand, pre-activation or
 *   logit was met on an active ray, in which case the caller re-renders the frame with
 *   mlpsp_render_tilecenter_f32 (rgb_wmma.cuh:260-272); the other words are reserved. */
size_t mlpsp_mfma_pack_bytes(int num_primitives);
int mlpsp_pack_mfma_weights(const float* W1, const float* b1, const float* W2, const float* b2, const float* W3,
                            const float* b3, int num_primitives, int use_bf16, void* packed_dev,
                            mlpsp_stream_t stream);
/* The same blocks from tensors STORED as fp16 -- the reference's inference export keeps MLP weights, biases and
 * feature attributes that way (scannet/checkpoints.py:317-381) and widens them to f32 when it loads them
 * (:299-314); here they are read as they are, with no f32 copy in between.  Every fp16 value is an f32 value, so
 * the blocks equal those of mlpsp_pack_mfma_weights on the widened tensors bit for bit. */
int mlpsp_pack_mfma_weights_half(const void* W1, const void* b1, const void* W2, const void* b2, const void* W3,
                                 const void* b3, int num_primitives, int use_bf16, void* packed_dev,
                                 mlpsp_stream_t stream);
int mlpsp_render_tilecenter_mfma(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                 const int32_t* order_dev, const int32_t* tile_offsets_dev, const float* freq_dev,
                                 const float* att_dev, const void* packed_dev, int num_primitives, int use_bf16,
                                 int width, int height, float threshold, float* out_rgb_dev, float* out_alpha_dev,
                                 int32_t* status_dev, int64_t* counters_dev, mlpsp_stream_t stream);

/* Matrix-core render with the gated feature channel (feat_slots 1, 4 or 5; channels <= 512).  No
 * counterpart in the reference, whose tensor-core kernel is RGB only; the feature semantics are those of
 * np_tile_kernels.cu:6036-6075 (feat += w * (base + sum_s g_s attr_s)) with this kernel's weights w.
 * The render kernel emits, per tile, the primitives that hit and their per-pixel coefficients w*g_s
 * rounded to fp16 into the workspace; a grouped fp16 GEMM (f32 accumulate) on the matrix cores then
 * forms the image from the fp16 attribute copy, whatever use_bf16 selects for the MLP.  out_feat_dev [B,C] is fully written.
 *
 * mlpsp_pack_mfma_feat: feat_attr f32 [N,S,C] ([N,C] for S = 1) -> operand copy (once per scene);
 * status_dev[0] = 1 if a value is not finite in fp16 (then use the f32 feature kernel).
 * num_pairs = length of order_dev = tile_offsets[num_tiles].  feat_slots = 0 renders RGB only and
 * ignores the feature and workspace arguments.  Workspace: mlpsp_feat_workspace_bytes(.., fp16_records = 1, ..);
 * status_dev[1] = 1 if its record pool ran out.  MLPSP_E_SCRATCH if the workspace is too small or not
 * 256-byte aligned.
 * stage: 0 = the whole frame; 1 = the render launch alone (RGB, alpha and the coefficient records in the workspace);
 * 2 = the feature product alone, over the records a stage-1 call with the same arguments left in the same workspace
 * (for timing the two launches apart; 1 and 2 need feat_slots != 0).  MLPSP_STAGE_STATUS_IS_CLEAR may be or-ed in:
 * the caller vouches that the 16 words at status_dev are zero already (it read them back as zero after the previous
 * call on this buffer), and the call queues no clear of them -- one launch less between the sort and the render
 * of a frame.
 * tile_ends_dev: NULL, or the ends of lists that lie in segments (see mlpsp_sort_tiles); num_pairs is then the
 * number of entries of order_dev, gaps included. */
#define MLPSP_STAGE_STATUS_IS_CLEAR 4
size_t mlpsp_mfma_feat_pack_bytes(int num_primitives, int feat_slots, int feat_channels);
int mlpsp_pack_mfma_feat(const float* feat_attr_dev, int num_primitives, int feat_slots, int feat_channels,
                         void* packed_feat_dev, int32_t* status_dev, mlpsp_stream_t stream);
/* mlpsp_pack_mfma_feat for attributes stored as fp16 [N,S,C] (the inference export): a pure re-ordering. */
int mlpsp_pack_mfma_feat_half(const void* feat_attr_dev, int num_primitives, int feat_slots, int feat_channels,
                              void* packed_feat_dev, int32_t* status_dev, mlpsp_stream_t stream);
int mlpsp_render_tilecenter_mfma_feat(const float* rays_o_dev, const float* rays_d_dev, const void* prim_records_dev,
                                      const int32_t* order_dev, const int32_t* tile_offsets_dev, int64_t num_pairs,
                                      const float* freq_dev, const float* att_dev, const void* packed_dev,
                                      int num_primitives, int use_bf16, const void* packed_feat_dev, int feat_slots,
                                      int feat_channels, float gating_beta, float gating_temp, int width, int height,
                                      float threshold, void* workspace_dev, size_t workspace_bytes,
                                      float* out_rgb_dev, float* out_alpha_dev, float* out_feat_dev,
                                      int32_t* status_dev, int64_t* counters_dev, int stage,
                                      const int32_t* tile_ends_dev, mlpsp_stream_t stream);

/* Weight and bias gradients of the per-primitive 72->32->32->4 MLP over a primitive-major CSR of hit records
 * = the Triton kernel _grouped_vjp (scannet/primitive_gemm.py:101-166, launched at :214-230).  Segment g covers
 * records [group_starts[g], min(group_starts[g] + segment, csr_offsets[group_primitives[g] + 1])) of primitive
 * group_primitives[g]; x6 [R,6] are the saved MLP inputs, grad4 [R,4] the adjoints of the four pre-activation
 * outputs, relu_masks [R,2] the saved activation masks (NULL: recompute them from the forward pass).
 * precision 0: IEEE f32 products and sums (fp32 MFMA), 1: fp16 operands, 2: bf16 operands, always with f32
 * accumulation over the segment; grad4 is multiplied by scale before rounding and the result divided by it.
 * partial_dev [num_groups, 3524] receives W1 (2304) | b1 (32) | W2 (1024) | b2 (32) | W3 (128) | b3 (4) per
 * segment.  segment must be a positive multiple of 32. */
int mlpsp_grouped_vjp(const float* x6_dev, const float* grad4_dev, const int32_t* relu_masks_dev,
                      const int64_t* csr_offsets_dev, const int64_t* group_primitives_dev,
                      const int64_t* group_starts_dev, int64_t num_groups, const float* freq_dev,
                      const float* att_dev, const float* W1, const float* b1, const float* W2, const float* b2,
                      const float* W3, int precision, float scale, int segment, float* partial_dev,
                      mlpsp_stream_t stream);

/* Sum of every primitive's segments = _reduce_partials (scannet/primitive_gemm.py:169-183): out_dev
 * [num_primitives, 3524] = sum over g in [group_offsets[p], group_offsets[p+1]) of partial_dev[g];
 * nonfinite_dev[0] is cleared and then set to 1 if any sum is NaN or infinite.  The sums are formed by chunks of
 * 32 consecutive segments and then per primitive (a fixed tree, so the result does not depend on scheduling),
 * which needs scratch rows behind the partial sums: partial_dev holds mlpsp_segment_reduce_rows(num_groups) rows
 * of 3524 floats, of which mlpsp_grouped_vjp fills the first num_groups.  group_primitives_dev as there. */
int64_t mlpsp_segment_reduce_rows(int64_t num_groups);
int mlpsp_reduce_partials(const float* partial_dev, const int64_t* group_primitives_dev,
                          const int64_t* group_offsets_dev, int64_t num_groups, int num_primitives, float* out_dev,
                          int32_t* nonfinite_dev, mlpsp_stream_t stream);
/* The same sums written straight into the six gradient tensors [N,32,72] [N,32] [N,32,32] [N,32] [N,4,32] [N,4]
 * (the reference splits and copies the packed rows afterwards, scannet/primitive_gemm.py:279); all 16-byte
 * aligned. */
int mlpsp_reduce_partials_split(const float* partial_dev, const int64_t* group_primitives_dev,
                                const int64_t* group_offsets_dev, int64_t num_groups, int num_primitives,
                                float* gW1_dev, float* gb1_dev, float* gW2_dev, float* gb2_dev, float* gW3_dev,
                                float* gb3_dev, int32_t* nonfinite_dev, mlpsp_stream_t stream);

/* Reverse compositing over saved forward records = primitive_records_reverse_kernel
 * (scannet/cuda/primitive_records.cuh:3-46; argument checks of its wrapper :48-74 are the caller's).
 * ids [R], pixel_offsets [num_pixels+1] (int64), x6 [R,6], raw [R,8] as written by mlpsp_records_emit;
 * grad_rgb [num_pixels,3], grad_t [num_pixels] = adjoint of the final transmittance.  Writes d4 [R,4], the
 * adjoint of the four pre-activation MLP outputs of every record, and ACCUMULATES (after clearing) the
 * gradients of positions [N,3], log-scales [N,3] and quaternions [N,4] that flow through the Gaussian
 * falloff, with f32 atomics (summation order not fixed).  raw, d4 and quats must be 16-byte aligned. */
int mlpsp_records_reverse(const int32_t* ids_dev, const int64_t* pixel_offsets_dev, const float* x6_dev,
                          const float* raw_dev, const float* log_scales_dev, const float* quats_dev,
                          const float* grad_rgb_dev, const float* grad_t_dev, int64_t num_pixels, int num_primitives,
                          float* d4_dev, float* grad_positions_dev, float* grad_log_scales_dev, float* grad_quats_dev,
                          mlpsp_stream_t stream);

/* The same reverse walk without atomics, for callers that go on to a primitive-major ordering of the records
 * anyway (the grouped weight gradients need one): writes d4 [R,4] as above and falloff_adjoint [R] =
 * dL/d(decay) * decay per record; mlpsp_geometry_gradients then forms the geometry gradients.  No counterpart
 * as a separate kernel in the reference (it is the first half of primitive_records_reverse_kernel). */
int mlpsp_records_reverse_adjoints(const int32_t* ids_dev, const int64_t* pixel_offsets_dev, const float* raw_dev,
                                   const float* grad_rgb_dev, const float* grad_t_dev, int64_t num_pixels,
                                   float* d4_dev, float* falloff_adjoint_dev, mlpsp_stream_t stream);

/* Second half of primitive_records_reverse_kernel (primitive_records.cuh:23-45) over records in primitive-major
 * order: primitive p owns rows [csr_offsets[p], csr_offsets[p+1]) of x6_sorted [R,6]; record_indices [R] (int64)
 * maps a row to its record, whose falloff_adjoint is read.  The rows are walked in the segments of
 * mlpsp_grouped_vjp (group_primitives / group_starts [num_groups], group_offsets [N+1], segment), one wavefront
 * per segment into partial_dev [num_groups, 16] (scratch), then summed per primitive.  Writes (not accumulates)
 * grad_positions [N,3], grad_log_scales [N,3], grad_quats [N,4]; no atomics, fixed summation order. */
int mlpsp_geometry_gradients(const int64_t* csr_offsets_dev, const int64_t* record_indices_dev,
                             const float* x6_sorted_dev, const float* falloff_adjoint_dev, const float* log_scales_dev,
                             const float* quats_dev, const int64_t* group_primitives_dev,
                             const int64_t* group_starts_dev, const int64_t* group_offsets_dev, int64_t num_groups,
                             int segment, int num_primitives, float* partial_dev, float* grad_positions_dev,
                             float* grad_log_scales_dev, float* grad_quats_dev, mlpsp_stream_t stream);

/* Streamed feature L1 loss over saved records = _stream_l1 (scannet/record_feature_loss.py:34-63, launched at
 * :66-89): for every pixel of the low-resolution target [target_height, target_width, channels] (f32, or fp16 if
 * target_is_half) the feature of its four bilinear source pixels is blended from their record lists
 * (ids [R], pixel_offsets [width*height+1] int64, raw [R,8], gates [R,4], attributes [N, slots, channels] with
 * slots 1, 4 or 5), combined with the weights of bilinear down-sampling (align_corners = false) and compared:
 * signs [target pixels, channels] int8 = sign(prediction - target), loss_partials [target pixels,
 * ceil(channels/128)] = per-block sums of |prediction - target| / (target pixels * channels), whose total is the
 * L1 loss.  prediction_dev (same shape as the target, f32) may be NULL. */
int mlpsp_stream_feature_l1(const int32_t* ids_dev, const int64_t* pixel_offsets_dev, const float* raw_dev,
                            const float* gates_dev, const float* attributes_dev, const void* target_dev,
                            int target_is_half, int width, int height, int target_width, int target_height,
                            int channels, int slots, int8_t* signs_dev, float* loss_partials_dev,
                            float* prediction_dev, mlpsp_stream_t stream);

/* Gradient of that loss with respect to the attributes = _feature_vjp + _feature_reduce
 * (scannet/record_feature_loss.py:114-185).  Records in primitive-major order: record_indices [R] (int64) maps a
 * row of the CSR (csr_offsets [N+1]) to its record, record_pixels [R] (int32) gives a record's pixel; segments as
 * for mlpsp_grouped_vjp.  mixed != 0 rounds both factors of every product to fp16 (f32 accumulation).
 * partial_dev [mlpsp_segment_reduce_rows(num_groups), slots, channels] is scratch (per-segment sums, then the
 * chunk sums of the per-primitive reduction), out_dev [N, slots, channels] the result.  group_order_dev (int64
 * [num_groups], a permutation, or NULL): the order in which the segments are launched; sorted by the segments' first
 * pixels, concurrent workgroups read neighbouring sign rows.  The result does not depend on it. */
int mlpsp_feature_attribute_gradients(const int8_t* signs_dev, const int64_t* record_indices_dev,
                                      const int32_t* record_pixels_dev, const float* raw_dev, const float* gates_dev,
                                      const int64_t* csr_offsets_dev, const int64_t* group_primitives_dev,
                                      const int64_t* group_starts_dev, const int64_t* group_offsets_dev,
                                      const int64_t* group_order_dev, int64_t num_groups, int num_primitives,
                                      int width, int height, int target_width,
                                      int target_height, int channels, int slots, int segment, int mixed,
                                      float* partial_dev, float* out_dev, mlpsp_stream_t stream);

/* Adjoint of the dense feature image with respect to the attributes = render_tiles_backward_featattr_tilecenter
 * (scannet/cuda/np_tile_kernels.cu:3531-3760, wrapper :6537-6620; called from _TileRenderWithFeatAutogradFn.backward,
 * scannet/cumodel.py:466-477): out[p, slot, c] = sum over the primitive's records of T * alpha * gate_slot *
 * grad_feat[record's pixel, c] (one slot: no gate; five slots: slot 0 has no gate).  The reference traverses the
 * frame again and adds with atomics; here the records saved by the records forward are used, in the layout of
 * mlpsp_feature_attribute_gradients (record_indices, record_pixels, csr_offsets, segments), and summed in a fixed
 * order.  grad_feat_dev [pixels, channels] f32; gates_dev may be NULL for one slot.  group_order_dev (int64
 * [num_groups], a permutation, or NULL) is the order in which the segments are launched: sorted by the segments' first
 * pixels, concurrent workgroups read neighbouring rows of grad_feat; the result does not depend on it.
 * partial_dev [mlpsp_segment_reduce_rows(num_groups), slots, channels] is scratch, out_dev [N, slots, channels]. */
int mlpsp_feature_dense_attribute_gradients(const float* grad_feat_dev, const int64_t* record_indices_dev,
                                            const int32_t* record_pixels_dev, const float* raw_dev,
                                            const float* gates_dev, const int64_t* csr_offsets_dev,
                                            const int64_t* group_primitives_dev, const int64_t* group_starts_dev,
                                            const int64_t* group_offsets_dev, const int64_t* group_order_dev,
                                            int64_t num_groups, int num_primitives, int channels, int slots, int segment,
                                            float* partial_dev, float* out_dev, mlpsp_stream_t stream);

/* Measurement aid, no counterpart in the reference: launches a kernel that does nothing but
 * v_mfma_f32_32x32x16_bf16 on register operands (2,048 workgroups x 4 wavefronts x iterations x 8
 * instructions) and returns the FLOPs it issues (-1 on error); time it on the stream to see what the
 * chip sustains next to the data-sheet peak.  sink_dev: one float, left untouched in practice. */
int64_t mlpsp_probe_mfma_bf16(int iterations, float* sink_dev, mlpsp_stream_t stream);

/* Measurement aid, no counterpart in the reference: how matrix-core, vector-ALU and transcendental instructions
 * share a SIMD's issue time.  256 workgroups of 16 wavefronts, one per CU, four wavefronts per SIMD (the render
 * kernel's occupancy); the wavefront of rank k on its SIMD (hardware id) runs roles[k] for window_us microseconds of
 * the constant-rate clock: 0 idle, 1 MFMA (16 v_mfma_f32_32x32x16_bf16 per batch, four independent accumulators),
 * 2 VALU (128 independent v_fma_f32), 3 transcendental (128 v_sin_f32), 4 mixed (16 x one MFMA followed by eight
 * independent v_fma_f32).  out_dev: 4096 records of 24 bytes {int64 batches, int64 core clocks, int32 role,
 * int32 simd}, one per wavefront.  Clocks per batch and SIMD = clocks / (batches x wavefronts of that role per SIMD).
 * Returns 0 or an MLPSP_E_* code.  sink_dev: one float, left untouched in practice. */
int mlpsp_probe_issue(const int32_t roles[4], int window_us, void* out_dev, float* sink_dev, mlpsp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MLPSP_H */
