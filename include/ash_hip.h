/*
 * ash_hip.h -- C ABI of libash_hip.so, the MI355X (gfx950) implementation of
 * torch-ash's two data-parallel hot paths:
 *
 *   1. the collision-free int32[dim] -> int32 index hash map
 *      (reference: the pybind class `HashMap`, ash/src/pybind.cpp:9-23,
 *       ash/src/hashmap.h:18-61, kernels in ash/src/hashmap_gpu.cuh);
 *   2. the sparse-dense grid trilinear query, forward / backward /
 *      double-backward (reference: ash/src/pybind.cpp:25-29, ash/src/grid.h:6-82,
 *      kernels in ash/src/grid.cu:68-451).
 *
 * Conventions
 *   - plain C, no torch types: device pointers are raw `void*` / typed pointers
 *     obtained from `Tensor.data_ptr()`; `stream` is a `hipStream_t` passed as
 *     `void*` (NULL = the null stream);
 *   - every function returns 0 on success, non-zero on failure; the message of
 *     the last failure on the calling thread is `ash_last_error()`;
 *   - nothing here allocates or frees device memory: table storage, outputs and
 *     temporaries are caller-owned buffers (the Python layer hands in torch
 *     tensors, so all device memory stays inside torch's caching allocator);
 *   - launches are asynchronous on `stream`; only `ash_map_status` /
 *     `ash_map_size` / `ash_map_counters` (which return host values)
 *     synchronise that stream, and are refused while it is being captured;
 *   - a map handle is not thread-safe; operations on one handle must be issued
 *     in order on one stream (as the reference issues them on the null stream);
 *   - calls on a map run on the map's device (ash_map_create's `device`); the
 *     calls that take tensors but no map (queries, convolution, surface
 *     extraction, depth integration) run on the device that holds their first
 *     tensor argument.  Either way the caller's current device is restored on
 *     return, and `stream` must belong to the device the call runs on.
 */
#ifndef ASH_HIP_H_
#define ASH_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ash_map ash_map_t;

/* Message of the last failing call on this thread ("" if none). */
const char* ash_last_error(void);

/* ABI version, bumped on incompatible changes. */
int ash_abi_version(void);

/* SHA-256 (hex) over the kernel sources this library was built from, as the
 * build computes it (names and contents of the .hip and .h files under
 * csrc/), or "unknown".  For benchmarks and tests to tell a library that does
 * not belong to the sources beside it.  No counterpart in the reference. */
const char* ash_source_fingerprint(void);

/* ------------------------------------------------------------------ hash map */

/* Storage needed for a table of `capacity` entries with `key_dim` int32 key
 * components (1..4, as ash/src/dispatch.h:50-68).
 *   table_bytes   : mandatory workspace (bucket array + device counters)
 *   general_bytes : optional second region, only needed once a key arrives
 *                   whose components do not fit the packed 64-bit code
 *                   (see ash_map_attach_general). */
int ash_map_workspace_bytes(int key_dim, int64_t capacity,
                            int64_t* table_bytes, int64_t* general_bytes);

/* Replaces `HashMap(key_dim, capacity, heap, device)` (ash/src/pybind.cpp:10,
 * ash/src/hashmap_impl.h:11-24).  `heap` is the caller-owned int32[capacity]
 * free list (the `_heap` state-dict buffer, ash/core.py:72-74); the map aliases
 * and mutates it exactly like the reference does.  `table_ws` is a 256-byte
 * aligned device buffer of at least `table_bytes` bytes.  The table is cleared
 * (heap := 0..capacity-1, size := 0) on `stream`; as after ash_map_clear, the
 * fill of the bucket array itself runs with the first call that needs it (a
 * streaming insert writes every bucket anyway and does not), so a new map,
 * like a cleared one, takes one call outside a graph capture before look-ups
 * on it can be captured. */
int ash_map_create(int key_dim, int64_t capacity, int32_t* heap,
                   void* table_ws, int64_t table_bytes, int device,
                   void* stream, ash_map_t** out);

/* Hands the map its second region: a 256-byte aligned device buffer of
 * general_bytes bytes, 20 per slot.  ash_map_workspace_bytes' general_bytes is
 * what `capacity` keys need at half load; a smaller buffer is taken as the
 * largest power of two of slots that fits (at least 64) -- enough for a caller
 * who attaches it ahead of time for keys that are not expected (a key that
 * finds such a region full is refused and counted like a key that finds the
 * map full).  Idempotent per handle: a second attach is an error. */
int ash_map_attach_general(ash_map_t* map, void* general_ws,
                           int64_t general_bytes, void* stream);

/* Releases the host-side handle only (device buffers are caller-owned). */
int ash_map_destroy(ash_map_t* map);

/* Replaces `HashMap::find` (ash/src/hashmap_gpu.cuh:163-208).
 * keys int32[n,key_dim] contiguous; indices int64[n]; masks uint8/bool[n].
 * Every output element is written: masks[i] = found, indices[i] = found ?
 * index : 0. */
int ash_map_find(ash_map_t* map, const int32_t* keys, int64_t n,
                 int64_t* indices, uint8_t* masks, void* stream);

/* Replaces the body of `SparseDenseGrid.query` (ash/grid.py:183-199: about ten
 * elementwise torch launches around one `find`) for a map with 3-d keys.
 * x float32[n,3] are positions in cell units and G = grid_dim cells per block
 * edge; per position, in fp32 and without fused multiply-add so that the
 * result equals the torch expression bit for bit:
 *   block = floor(x / G), inner = x - block * G, offsets = inner - floor(inner),
 *   cell_indices = ix + G*iy + G*G*iz with i = (int)inner,
 *   (grid_indices, masks) = find((int)block).
 * Right at a block boundary fp32 rounding can take `inner` out of [0, G)
 * (negative, or exactly G); such positions are moved to the neighbouring
 * block so that cell indices stay in range.  Every output element is written. */
int ash_grid_query(ash_map_t* map, const float* x, int64_t n, int grid_dim,
                   int64_t* grid_indices, int64_t* cell_indices, float* offsets,
                   uint8_t* masks, void* stream);

/* Stands for the body of `SparseDenseGrid.spatial_init_` (ash/grid.py:133-152):
 * for every position `cells[i]` (fp32, cell units) the block
 * floor(cells[i] / grid_dim) and its neighbours within `dilation` blocks
 * (offsets -dilation..dilation per axis if `bidirectional`, else 0..dilation)
 * are inserted as int3 keys.  Blocks with a coordinate outside
 * [bound_lo, bound_hi] are skipped, and so are all candidates of a position
 * whose own block is outside (the reference's grids_in_bound, applied before
 * and after the expansion).  The reference de-duplicates the (2r+1)^3 N
 * candidate rows through a scratch HashSet; here the candidates are generated
 * in registers and the table absorbs the duplicates.
 * Afterwards every touched block (new or already stored) has touched[index] = 1
 * and its coordinates at coords[3*index..]; both are caller-owned arrays of
 * `capacity` rows, `touched` zero on entry for the caller to tell this batch's
 * blocks.  heads_scratch: device temporary of 64 + 3 n int32 (one block per run
 * of consecutive positions in the same block).  Keys refused for lack of
 * capacity are counted as by insert_keys. */
int ash_grid_activate(ash_map_t* map, const float* cells, int64_t n,
                      int grid_dim, int dilation, int bidirectional,
                      int bound_lo, int bound_hi, uint8_t* touched,
                      int32_t* coords, int32_t* heads_scratch, void* stream);

/* ash_grid_activate for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops that must not reach hipMalloc, harnesses
 * that forbid it): same arguments, same result, but the list of run heads lives
 * in a device array inside the library instead of `heads_scratch`, and the call
 * allocates nothing on the host or the device.  No counterpart in the
 * reference.
 *   - at most ASH_ACTIVATE_STATIC_MAX_POSITIONS positions per call (a 1024 x
 *     1024 depth image); more is an error, nothing is launched;
 *   - the array (64 + 3 * ASH_ACTIVATE_STATIC_MAX_POSITIONS int32, 12.6 MB) is
 *     held by every device that loads the library until the process ends;
 *   - all calls on one device share it, on whatever map or stream: two calls
 *     whose work overlaps in time on one device race.  Issue them on one
 *     stream, or order the streams with events. */
#define ASH_ACTIVATE_STATIC_MAX_POSITIONS (1 << 20)
int ash_grid_activate_static(ash_map_t* map, const float* cells, int64_t n,
                             int grid_dim, int dilation, int bidirectional,
                             int bound_lo, int bound_hi, uint8_t* touched,
                             int32_t* coords, void* stream);

/* ash_grid_activate straight from world positions and without a scratch
 * buffer: `positions` fp32[n,3] in world units, cell units = (position -
 * origin) / cell_size evaluated as torch evaluates that expression on the
 * device (a subtraction, then a multiplication by the fp32 reciprocal);
 * `origin` fp32[3] ON THE DEVICE or NULL, cell_size 1 with a NULL origin for
 * positions that are in cell units already.  Stands for
 * `transform_world_to_cell` + the body of `spatial_init_` (ash/grid.py:121-159)
 * in two launches: every workgroup finds the run heads among its own 128
 * positions, so there is no list of heads, no counter to clear and nothing to
 * allocate.  Same blocks, flags and coordinates as ash_grid_activate. */
int ash_grid_activate_positions(ash_map_t* map, const float* positions, int64_t n,
                                const float* origin, float cell_size, int grid_dim,
                                int dilation, int bidirectional, int bound_lo,
                                int bound_hi, uint8_t* touched, int32_t* coords,
                                void* stream);

/* After ash_grid_activate: the rows whose flag is set in `touched`, in
 * ascending order, to out_indices int64[capacity] and their block coordinates
 * to out_coords int32[capacity, 3]; the flags are cleared and the count is left
 * in the table's counters (out[5] of ash_map_counters), so that the
 * read-back that follows an activation anyway also sizes the result -- instead
 * of a `nonzero` over the flags with a read-back of its own.  Tables of up to
 * ASH_COLLECT_MAX_BLOCKS rows; `touched` 4-byte aligned.  No counterpart in the
 * reference. */
#define ASH_COLLECT_MAX_BLOCKS (1 << 20)
int ash_grid_collect_touched(ash_map_t* map, uint8_t* touched, const int32_t* block_coords,
                             int64_t* out_indices, int32_t* out_coords, void* stream);

/* Stands for `project_points_to_rgbd` plus the fusion arithmetic of
 * `fuse_frame` in the reference's TSDF demo (demo/rgbd_fusion.py:76-110,
 * 216-254), which are torch expressions around
 * embeddings[grid_indices, cell_indices]: every cell of the `n_blocks` listed
 * blocks is projected into the depth image (world = (block * grid_dim + cell)
 * * cell_size [+ origin], camera = extrinsic * world, pixel = round(K * camera
 * / z)), and its embedding row is updated in place with the running weighted
 * mean: channel 0 = truncated signed distance, channels 1..3 = colour when
 * `color` is given (then embedding_dim >= 5), last channel = weight.
 * embeddings fp32 [num_embeddings, grid_dim^3, embedding_dim]; grid_indices
 * int64[n_blocks] rows of it, grid_coords int32[n_blocks,3]; intrinsic 3x3 and
 * extrinsic 4x4 row-major fp32 ON THE DEVICE; origin: host float[3] or NULL;
 * depth fp32[height,width] (0 = no reading), color fp32[height,width,3] or
 * NULL. */
int ash_grid_integrate_depth(float* embeddings, int64_t num_embeddings,
                             int grid_dim, int embedding_dim,
                             const int64_t* grid_indices,
                             const int32_t* grid_coords, int64_t n_blocks,
                             float cell_size, const float* origin,
                             const float* intrinsic, const float* extrinsic,
                             const float* depth, const float* color, int height,
                             int width, float trunc, float depth_max,
                             void* stream);

/* ash_grid_integrate_depth over the listing that the latest
 * ash_grid_collect_touched on `map` left (out_indices / out_coords of that
 * call, both of `capacity` rows), whose length is read on the device from the
 * table's counters: no host value depends on the activation, so a frame of a
 * fusion loop (activate, list, integrate) needs no read-back at all.  A fixed
 * grid strides over the listed blocks' cells.  Same arithmetic and arguments
 * otherwise.  No counterpart in the reference, whose loop sizes tensors by the
 * number of touched blocks (demo/rgbd_fusion.py:216-254). */
int ash_grid_integrate_depth_touched(ash_map_t* map, float* embeddings,
                                     int64_t num_embeddings, int grid_dim,
                                     int embedding_dim, const int64_t* grid_indices,
                                     const int32_t* grid_coords, float cell_size,
                                     const float* origin, const float* intrinsic,
                                     const float* extrinsic, const float* depth,
                                     const float* color, int height, int width,
                                     float trunc, float depth_max, void* stream);

/* ash_grid_integrate_depth over every row whose flag an activation has set in
 * `touched` (uint8[capacity]; block coordinates at coords[3*row..], as
 * ash_grid_activate leaves them), without a listing in between: the kernel
 * looks at the flags itself, takes them down and updates the cells of the
 * flagged blocks.  With ash_grid_activate_positions a frame of a fusion loop
 * is three launches, none of which waits for the host.  Same arithmetic as
 * ash_grid_integrate_depth.  No counterpart in the reference. */
int ash_grid_integrate_depth_flagged(ash_map_t* map, float* embeddings,
                                     int64_t num_embeddings, int grid_dim,
                                     int embedding_dim, uint8_t* touched,
                                     const int32_t* coords, float cell_size,
                                     const float* origin, const float* intrinsic,
                                     const float* extrinsic, const float* depth,
                                     const float* color, int height, int width,
                                     float trunc, float depth_max, void* stream);

/* Replaces `ray_find_near_far` (ash/src/sampler.cu:7-121, pybind.cpp:35): per
 * ray, march from t_min in steps of half a block while inside the box
 * [bbox_min, bbox_max] and report the range [near, far] that contains active
 * blocks; near = -1 when none is met.  Origins / directions fp32[n,3] in cell
 * units, bbox_min / bbox_max fp32[3] on the device.  `t_step` is accepted and
 * unused, as in the reference. */
int ash_ray_find_near_far(ash_map_t* map, const float* ray_origins,
                          const float* ray_directions, const float* bbox_min,
                          const float* bbox_max, int64_t n, float t_min,
                          float t_max, float t_step, float grid2cell_multiplier,
                          float* ray_nears, float* ray_fars, void* stream);

/* Replaces the two launches of `ray_sample` (ash/src/sampler.cu:122-294,
 * pybind.cpp:36-37).  Allocation pass: counts int64[n] receives the number of
 * samples per ray (prefix and the outputs NULL).  The caller forms the
 * inclusive prefix sum and allocates; assignment pass: counts NULL, prefix
 * int64[n], ray_indices int64[total], t_nears / t_fars fp32[total]. */
int ash_ray_sample(ash_map_t* map, const float* ray_origins,
                   const float* ray_directions, const float* ray_nears,
                   const float* ray_fars, int64_t n, int64_t max_samples_per_ray,
                   float grid2cell_multiplier, int64_t* counts,
                   const int64_t* prefix, int64_t* ray_indices, float* t_nears,
                   float* t_fars, void* stream);

/* The same result with one march instead of two (no counterpart in the
 * reference, whose second launch repeats the march of the first).  staged:
 * the allocation pass, which also keeps the first `stride` samples of every ray
 * in stage fp32[n * stride * 2] (8-byte aligned).  compact: the assignment
 * pass as a copy out of `stage`; valid when no ray has more than `stride`
 * samples (counts tells; max_samples_per_ray + 2 always suffices), otherwise
 * run the assignment pass of ash_ray_sample. */
int ash_ray_sample_staged(ash_map_t* map, const float* ray_origins,
                          const float* ray_directions, const float* ray_nears,
                          const float* ray_fars, int64_t n, int64_t max_samples_per_ray,
                          float grid2cell_multiplier, int64_t* counts, float* stage,
                          int64_t stride, void* stream);
int ash_ray_sample_compact(const int64_t* counts, const int64_t* prefix, const float* stage,
                           int64_t stride, int64_t n, int64_t* ray_indices, float* t_nears,
                           float* t_fars, void* stream);

/* Replaces `HashMap::insert_keys` (ash/src/hashmap_gpu.cuh:211-247).  New keys
 * pop one index each from the heap; duplicates (in the table or within the
 * batch) are ignored.  Keys beyond `capacity` are dropped and counted
 * (ash_map_status), where the reference reads past the heap. */
int ash_map_insert_keys(ash_map_t* map, const int32_t* keys, int64_t n,
                        void* stream);

/* 1 when ash_map_insert needs the `assigned` temporary for these rows. */
int ash_map_insert_needs_scratch(int n_values, const int64_t* row_bytes);

/* Replaces `HashMap::insert(keys, values, external_values)`
 * (ash/src/hashmap_gpu.cuh:249-313).  For value tensor j, the row
 * src[j] + i*row_bytes[j] of every newly inserted key i is copied to
 * dst[j] + index*row_bytes[j].  `assigned` is an int32[n] device temporary,
 * required (non-NULL) only when ash_map_insert_needs_scratch(...) is 1. */
int ash_map_insert(ash_map_t* map, const int32_t* keys, int64_t n,
                   int n_values, const void* const* src, void* const* dst,
                   const int64_t* row_bytes, int32_t* assigned, void* stream);

/* Streaming variant of ash_map_insert_keys / ash_map_insert for batches of
 * the order of the table itself (same reference functions,
 * ash/src/hashmap_gpu.cuh:211-313, same resulting map): the batch is split by
 * bucket range in two coalesced passes and each range of 512 buckets is then
 * built in LDS by one workgroup and written back whole, so no global atomic is
 * issued per key.  Inputs it cannot place that way (unpackable keys, piles of
 * duplicates, an exhausted heap) are finished by the per-key kernel inside the
 * same call.
 *   ash_map_bulk_workspace_bytes: *bytes = size of the device workspace for
 *   `n` keys with these value rows, 0 when the path does not apply (fewer than
 *   4096 keys, rows that need `assigned`, a table of more than 2^25 buckets);
 *   *worthwhile (optional) = 1 when n is large enough relative to the table
 *   for the streaming path to be the faster one.
 *   ash_map_insert_bulk: n_values may be 0 (keys only).  The workspace is
 *   256-byte aligned, caller-owned and free again when the call's work on
 *   `stream` has finished. */
int ash_map_bulk_workspace_bytes(ash_map_t* map, int64_t n, int n_values,
                                 const int64_t* row_bytes, int64_t* bytes,
                                 int* worthwhile);
int ash_map_insert_bulk(ash_map_t* map, const int32_t* keys, int64_t n,
                        int n_values, const void* const* src, void* const* dst,
                        const int64_t* row_bytes, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* Replaces `HashMap::erase` (ash/src/hashmap_gpu.cuh:316-351): found keys are
 * removed and their indices pushed back on the heap; duplicates inside the
 * batch erase once. */
int ash_map_erase(ash_map_t* map, const int32_t* keys, int64_t n, void* stream);

/* Streaming variant of ash_map_erase for batches of the order of the table
 * (same reference function, ash/src/hashmap_gpu.cuh:316-351, same resulting
 * map): the batch is split by bucket range as for ash_map_insert_bulk, and each
 * range of 512 buckets is taken into LDS by one workgroup, which frees the
 * slots of its keys there and writes the range back; the heap counter moves
 * once per workgroup instead of one global compare-and-swap per key.
 *   ash_map_erase_bulk_query: *bytes = size of the device workspace for `n`
 *   keys (0 when the path does not apply, as for ash_map_bulk_workspace_bytes
 *   without value rows); *worthwhile (optional) = 1 when n is large enough
 *   relative to the table for this path to be the faster one.
 *   ash_map_erase_bulk: workspace as for ash_map_insert_bulk. */
int ash_map_erase_bulk_query(ash_map_t* map, int64_t n, int64_t* bytes, int* worthwhile);
int ash_map_erase_bulk(ash_map_t* map, const int32_t* keys, int64_t n, void* workspace,
                       int64_t workspace_bytes, void* stream);

/* `HashMap::insert_keys` / `HashMap::insert` (ash/src/hashmap_gpu.cuh:211-313)
 * as one call that keeps the table in order by itself -- what a binding with
 * the reference's nine methods (ash/src/pybind.cpp:9-23) calls:
 *   1. if an erase or refused keys may have left tombstones, it looks at the
 *      counters and re-places the entries when too few empty slots remain
 *      (ash_map_should_rebuild / ash_map_rebuild);
 *   2. it takes the streaming path (ash_map_insert_bulk) when the batch is large
 *      enough relative to the table, else the per-key kernel, with `scratch` as
 *      the workspace of either (`policy` overrides the choice);
 *   3. it reads the counters, or -- streaming path, a landing place set with
 *      ash_map_set_staging, no key of the batch handed to the per-key kernel --
 *      queues their read-back behind the insert and returns without waiting
 *      for it (ash_map_counters picks it up).
 * Returns ASH_NEEDS_GENERAL (and inserts everything else) when keys of the
 * batch do not fit the packed code and no second region is attached: attach
 * one and issue the same call again.  n_values may be 0 (keys only).
 * ash_map_insert_scratch_bytes gives the size of `scratch` (256-byte aligned
 * device memory, free again when the call's work on `stream` has finished) for
 * the call that follows it.  On a stream that is being captured the call only
 * queues launches (no upkeep, no look at the counters): refused keys and keys
 * waiting for the second region stay in the counters.  `staging` as for
 * ash_map_counters. */
enum { ASH_STREAMING_AUTO = 0, ASH_STREAMING_ALWAYS = 1, ASH_STREAMING_NEVER = 2 };
enum { ASH_NEEDS_GENERAL = 2 };
int ash_map_insert_scratch_bytes(ash_map_t* map, int64_t n, int n_values,
                                 const int64_t* row_bytes, int policy, int64_t* bytes);
int ash_map_insert_auto(ash_map_t* map, const int32_t* keys, int64_t n, int n_values,
                        const void* const* src, void* const* dst, const int64_t* row_bytes,
                        void* scratch, int64_t scratch_bytes, int policy, int32_t* staging,
                        void* stream);

/* `HashMap::erase` (ash/src/hashmap_gpu.cuh:316-351) with the choice between
 * ash_map_erase and ash_map_erase_bulk made here; scratch as above. */
int ash_map_erase_scratch_bytes(ash_map_t* map, int64_t n, int policy, int64_t* bytes);
int ash_map_erase_auto(ash_map_t* map, const int32_t* keys, int64_t n, void* scratch,
                       int64_t scratch_bytes, int policy, void* stream);

/* Step 1 of ash_map_insert_auto on its own, for the entry points that insert
 * without it (ash_grid_activate*): call it before them.  `scratch` is only
 * needed by a map with a second region (ash_map_insert_scratch_bytes with
 * n = 0 sizes it).  Does nothing on a stream that is being captured. */
int ash_map_upkeep(ash_map_t* map, int64_t incoming, void* scratch, int64_t scratch_bytes,
                   int32_t* staging, void* stream);

/* Replaces `HashMap::clear` (ash/src/hashmap_gpu.cuh:354-358,
 * ash/src/hashmap_impl.h:26-33).  Counters, heap and the second region are
 * reset on `stream` at once (the heap array is rewritten to 0..capacity-1 only
 * when ash_map_erase or ash_map_load has written to it since it was last in
 * that state: inserts only read it, and nothing but this library may write to
 * it while the map lives; while it is in that state listings read the log of
 * stored keys only below the size, so the log is left as it is and emptied
 * beyond the size by the first erase); the fill of the bucket array runs with the next
 * call that reads or updates the table, on that call's stream, and not at all
 * when that call is an ash_map_insert_bulk, which rewrites every bucket.  A
 * call whose stream is being captured refuses to run that pending fill (the
 * graph would empty the table at every replay). */
int ash_map_clear(ash_map_t* map, void* stream);

/* Host read-back of the device counters; always a copy from the device, which
 * synchronises `stream`.
 *   out[0] size (= heap counter, ash/src/hashmap_gpu.cuh:157)
 *   out[1] keys dropped because the map was full (since the last clear)
 *   out[2] tombstoned slots
 *   out[3] keys that are waiting for ash_map_attach_general (re-issue the
 *          insert after attaching; the counter is reset by the attach)
 *   out[4] pairs refused by ash_map_load: duplicate keys, indices or heap
 *          entries outside 0 .. capacity-1 */
int ash_map_status(ash_map_t* map, int64_t out[5], void* stream);

/* The same counters as the handle knows them, plus out[5] = rows listed by the
 * latest ash_grid_collect_touched and out[6] = entries that live in the second
 * region.  The handle follows every call that changes them: after a clear they
 * are known to be zero, after ash_map_insert_auto they have been read (or are
 * on their way, see there) -- only when neither holds are they copied from the
 * device, which synchronises `stream`.  `staging`: eight int32 of page-locked
 * host memory of the calling thread's for that copy, or NULL (pageable memory:
 * about twice the latency).  No counterpart in the reference, whose `size()`
 * synchronises every time (ash/src/hashmap_gpu.cuh:157). */
int ash_map_counters(ash_map_t* map, int32_t* staging, int64_t out[7], void* stream);
/* 1 while the read-back that a streaming ash_map_insert_auto queued has not
 * been looked at yet. */
int ash_map_counters_pending(ash_map_t* map);
/* 1 and *size when the size is known without a copy from the device (waits for
 * a queued read-back if there is one), 0 when it is not, -1 on failure. */
int ash_map_known_size(ash_map_t* map, int64_t* size);
/* Gives the map sixteen int32 of page-locked host memory of its own (NULL takes
 * them away again): the landing place of the read-back that a streaming
 * ash_map_insert_auto queues behind itself.  Must outlive the map or be taken
 * away first. */
int ash_map_set_staging(ash_map_t* map, int32_t* staging);

/* Replaces `HashMap::size` (ash/src/hashmap_gpu.cuh:157); synchronises. */
int ash_map_size(ash_map_t* map, int64_t* size, void* stream);

/* Replaces `HashMap::items` (ash/src/hashmap_gpu.cuh:360-405): writes the
 * live (key, index) pairs in unspecified order.  keys_out int32[n_expected,
 * key_dim], indices_out int64[n_expected]; n_expected must be the current
 * size (rows beyond it are never written). */
int ash_map_items(ash_map_t* map, int32_t* keys_out, int64_t* indices_out,
                  int64_t n_expected, void* stream);

/* Whether the next ash_map_items lists entry i under index i (*dense = 1):
 * while nothing has been erased or loaded since the map was created or
 * cleared and no key lives in the second region, the indices in use are
 * 0 .. size-1 (a new key takes heap[counter++], ash/src/hashmap_gpu.cuh:226-231,
 * from a heap in its initial order, ash/src/hashmap_impl.h:26-33), and the
 * listing follows them.  A binding can then take the value rows of the listed
 * entries as the first `size` rows of every value tensor instead of gathering
 * them by index (`values[name][indices]`, ash/hashmap.py:138-146).  Host-side
 * state only, no synchronisation.  No counterpart in the reference. */
int ash_map_items_in_index_order(ash_map_t* map, int* dense);

/* Replaces `HashMap::load_states` (ash/src/hashmap_gpu.cuh:407-450): the map
 * is emptied, then (keys[i] -> indices[i]) are stored, size := n and the heap
 * := heap_src (skipped when heap_src is NULL or already the map's heap). */
int ash_map_load(ash_map_t* map, const int32_t* keys, const int64_t* indices,
                 int64_t n, const int32_t* heap_src, void* stream);

/* Erasing from buckets that have been full, and refusing keys of an overfull
 * batch, leaves tombstoned slots behind.  `ash_map_should_rebuild` (host
 * arithmetic only) says whether, with `size` live entries, `tombstones`
 * tombstones and `incoming` keys about to arrive, fewer than a fifth of the
 * slots would stay empty.  `ash_map_rebuild` then re-places the `n` = size live
 * (key, index) pairs into an emptied table; indices, heap and size are
 * untouched.  A map without a second region puts them back from its log of
 * stored keys and needs no scratch (both pointers may be NULL); with one,
 * keys_scratch int32[n,key_dim] and indices_scratch int64[n] are device
 * temporaries.  ash_map_insert_auto / ash_map_upkeep do both by themselves.
 * No counterpart in the reference, whose container recycles slots itself. */
int ash_map_should_rebuild(ash_map_t* map, int64_t size, int64_t tombstones,
                           int64_t incoming);
int ash_map_rebuild(ash_map_t* map, int32_t* keys_scratch,
                    int64_t* indices_scratch, int64_t n, void* stream);

/* Generic row scatter used by the wide-row path of ash_map_insert, exported
 * because the Python layer reuses it: dst[assigned[i]] = src[i] for
 * assigned[i] >= 0. */
int ash_scatter_rows(const void* src, void* dst, const int32_t* assigned,
                     int64_t n, int64_t row_bytes, void* stream);

/* The gather behind `HashMap.find(return_values=True)` /
 * `HashMap.items(return_values=True)` (ash/hashmap.py:87-95,138-146: the
 * reference indexes every value tensor with the returned indices, one torch
 * launch per tensor): dst[v][i] = src[v][indices[i]] for up to four tensors in
 * one launch.  Rows of tensor v are row_bytes[v] bytes (a multiple of 4), the
 * source has src_rows[v] rows; an index outside the source gives a zero row.
 * dst[v] holds n rows.  indices == NULL stands for 0, 1, .., n-1 (what a
 * listing holds while ash_map_items_in_index_order says so): the first n rows
 * are copied.  Runs on the device that holds the first source tensor. */
int ash_gather_rows(int n_values, const void* const* src, void* const* dst,
                    const int64_t* row_bytes, const int64_t* src_rows,
                    const int64_t* indices, int64_t n, void* stream);

/* -------------------------------------------------------- trilinear queries */

enum { ASH_INTERP_LINEAR = 0, ASH_INTERP_SMOOTH_STEP = 1 };
enum { ASH_F32 = 0, ASH_F64 = 1 };

/* Operands shared by the three query entry points (ash/src/grid.h:6-82):
 *   embeddings   scalar[B, M, E]   (M = cells per block, E <= 16)
 *   offsets      float32[N, 3]     (always fp32, ash/src/grid.cu:71)
 *   grid_indices int64[N], cell_indices int64[N], masks uint8/bool[N]
 *                (B and M are below 2^31 and only the low 32 bits of an index
 *                are read; what a masked query holds there is read and dropped)
 *   lut_grid_nb2grid_idx int64[B, 8]  (-1 = missing neighbour block)
 *   lut_cell_nb2cell_idx int64[M, 8], lut_cell_nb2grid_nb int64[M, 8] */
typedef struct ash_query_args {
    const void* embeddings;
    const float* offsets;
    const int64_t* grid_indices;
    const int64_t* cell_indices;
    const uint8_t* masks;
    const int64_t* lut_grid_nb2grid_idx;
    const int64_t* lut_cell_nb2cell_idx;
    const int64_t* lut_cell_nb2grid_nb;
    int64_t num_queries;    /* N */
    int64_t num_embeddings; /* B */
    int64_t cells_per_grid; /* M */
    int64_t embedding_dim;  /* E */
    int32_t interpolation;  /* ASH_INTERP_* */
    int32_t dtype;          /* ASH_F32 / ASH_F64: dtype of embeddings & grads */
} ash_query_args;

/* Replaces `query_forward` (ash/src/grid.cu:68-175).  output scalar[N, E];
 * every row is written (zeros for masked-out queries and for queries with a
 * missing neighbour block, ash/src/grid.cu:84-86,109-111). */
int ash_query_forward(const ash_query_args* a, void* output, void* stream);

/* Replaces the linear / smooth_step branch of `SparseDenseGrid.forward`
 * (ash/grid.py:201-238: world -> cell units, ash/grid.py:753,852, `query`,
 * ash/grid.py:183-199, then `query_forward`, ash/src/grid.cu:68-175) in one
 * kernel: x float32[N,3] positions -> output scalar[N, E] and masks
 * uint8/bool[N] (= block is active).  Positions become cell units as
 * (x - origin) * (1.0f / cell_size) in fp32 -- what torch computes on the
 * device for `(x - origin) / cell_size` -- with origin float32[3] on the
 * device or NULL for none; origin NULL and cell_size 1 leave x as it is, and
 * the results are then bit for bit what ash_grid_query followed by
 * ash_query_forward give.  Of
 * `tables` the embeddings, the three neighbour tables, the sizes (num_queries
 * = N, cells_per_grid = grid_dim^3), interpolation and dtype are used; its
 * per-query arrays are not read and may be NULL.  grid_indices int64[N],
 * cell_indices int64[N] and offsets float32[N,3] are the intermediate results
 * a later backward pass needs: pass all three to have them written, or three
 * NULLs to skip them (inference).  `map` must have 3-d keys and live on the
 * device of the embeddings. */
int ash_grid_forward(ash_map_t* map, const float* x, const float* origin, float cell_size,
                     int grid_dim, const ash_query_args* tables, void* output, uint8_t* masks,
                     int64_t* grid_indices, int64_t* cell_indices, float* offsets,
                     void* stream);

/* Replaces `query_backward_forward` (ash/src/grid.cu:177-307).
 * z scalar[N, E]; grad_embeddings scalar[B, M, E] (zero-filled here, then
 * accumulated); grad_offsets scalar[N, 3] (every row written).  One of the two
 * outputs may be NULL: it is then not computed (for grad_embeddings that saves
 * the dense zero fill and all atomics), which is what an autograd caller wants
 * when only one gradient was requested. */
int ash_query_backward_forward(const ash_query_args* a, const void* z,
                               void* grad_embeddings, void* grad_offsets,
                               void* stream);

/* Replaces `query_backward_backward` (ash/src/grid.cu:309-451).
 * grad_grad_offsets scalar[N,3], z scalar[N,E]; outputs grad_z scalar[N,E]
 * (every row written) and grad_embeddings scalar[B,M,E] (zero-filled here).
 * As in the reference the incoming grad_grad_embeddings is not used and the
 * offsets gradient is identically zero (ash/src/grid.cu:417-426); the caller
 * produces that zero tensor itself.  One of grad_z / grad_embeddings may be
 * NULL and is then not computed. */
int ash_query_backward_backward(const ash_query_args* a,
                                const void* grad_grad_offsets, const void* z,
                                void* grad_z, void* grad_embeddings,
                                void* stream);

/* The two gradient calls above with grad_embeddings added to instead of
 * zero-filled: the caller passes a gradient that already holds the other
 * contributions to the same embeddings (it must not be NULL).  No counterpart
 * in the reference, which zero-fills a new dense tensor in every call and
 * leaves the sum of two such tensors to autograd: a training step with a value
 * loss and a gradient-norm loss then pays two dense fills and one dense add
 * that this variant saves. */
int ash_query_backward_forward_accumulate(const ash_query_args* a, const void* z,
                                          void* grad_embeddings, void* grad_offsets,
                                          void* stream);
int ash_query_backward_backward_accumulate(const ash_query_args* a,
                                           const void* grad_grad_offsets, const void* z,
                                           void* grad_z, void* grad_embeddings,
                                           void* stream);

/* Replaces `convolution_forward` (ash/src/grid.cu:948-1043, pybind.cpp:33).
 * inputs / outputs scalar[num_embeddings, cells_per_grid, embedding_dim];
 * weights scalar[num_cell_nbs, embedding_dim] (one weight per window tap and
 * channel); masks bool[>= num_grids * cells_per_grid]; grid_indices
 * int64[num_grids] (rows of the listed blocks), cell_indices
 * int64[cells_per_grid]; the three neighbour tables as for the queries but over
 * the convolution window: lut_grid_nb2grid_idx int64[num_embeddings,
 * num_grid_nbs], lut_cell_nb2cell_idx / lut_cell_nb2grid_nb
 * int64[cells_per_grid, num_cell_nbs].  `outputs` is zero-filled here; rows of
 * blocks that are not listed stay zero. */
int ash_convolution_forward(const void* inputs, const void* weights,
                            const uint8_t* masks, const int64_t* grid_indices,
                            const int64_t* cell_indices,
                            const int64_t* lut_grid_nb2grid_idx,
                            const int64_t* lut_cell_nb2cell_idx,
                            const int64_t* lut_cell_nb2grid_nb, void* outputs,
                            int64_t num_grids, int64_t num_embeddings,
                            int64_t cells_per_grid, int64_t embedding_dim,
                            int64_t num_cell_nbs, int64_t num_grid_nbs,
                            int32_t dtype, void* stream);

/* ash_convolution_forward with one scratch byte per block, `listed`
 * uint8[num_embeddings] (uninitialised): the library marks the listed blocks
 * there and clears only the rows of the others, and the kernel that serves
 * cube windows over cubic blocks writes every cell of the blocks it is given,
 * zeros where the plain call leaves the cleared value.  Same result; saves
 * most of the dense clear when most blocks are listed.  Shapes that kernel does
 * not take run exactly as in the plain call.  No counterpart in the reference
 * (at::zeros_like, ash/src/grid.cu:1010). */
int ash_convolution_forward_listed(const void* inputs, const void* weights,
                                   const uint8_t* masks, const int64_t* grid_indices,
                                   const int64_t* cell_indices,
                                   const int64_t* lut_grid_nb2grid_idx,
                                   const int64_t* lut_cell_nb2cell_idx,
                                   const int64_t* lut_cell_nb2grid_nb, void* outputs,
                                   int64_t num_grids, int64_t num_embeddings,
                                   int64_t cells_per_grid, int64_t embedding_dim,
                                   int64_t num_cell_nbs, int64_t num_grid_nbs,
                                   int32_t dtype, uint8_t* listed, void* stream);

/* Replace the two launches of `isosurface_extraction` (ash/src/grid.cu:453-602,
 * pybind.cpp:30; the reference counts, allocates and runs the same kernel again
 * to fill).  sdfs / weights scalar[num_embeddings, cells_per_grid];
 * grid_indices int64[num_grids]; grid_coords_table int32[num_embeddings, 3];
 * cell_coords_table int32[cells_per_grid, 3]; the three 8-entry neighbour
 * tables of the queries.
 *
 * classify: flags uint8[num_embeddings * cells_per_grid] (no initialisation)
 * receives, for every cell of the listed rows, bit d set when the field crosses
 * iso_value on the cell's +x/+y/+z edge (d = 0, 1, 2) and both ends weigh at
 * least weight_thr; a missing neighbour block ends a cell's scan as in the
 * reference.  workspace (device int32, as many as
 * ash_isosurface_workspace_ints returns, no initialisation): [0] = number of
 * points, the rest is carried to the second call.
 *
 * points: after the caller has read workspace[0] and allocated positions
 * fp32[n_points, 3] (cell units); the points come in the order of the listing,
 * the same on every run. */
int64_t ash_isosurface_workspace_ints(int64_t num_grids, int64_t cells_per_grid);
int ash_isosurface_classify(const void* sdfs, const void* weights, const int64_t* grid_indices,
                            const int64_t* lut_grid_nb2grid_idx,
                            const int32_t* cell_coords_table,
                            const int64_t* lut_cell_nb2cell_idx,
                            const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                            int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                            float iso_value, float weight_thr, int32_t dtype, uint8_t* flags,
                            int32_t* workspace, void* stream);
int ash_isosurface_points(const void* sdfs, const int64_t* grid_indices,
                          const int32_t* grid_coords_table,
                          const int64_t* lut_grid_nb2grid_idx,
                          const int32_t* cell_coords_table,
                          const int64_t* lut_cell_nb2cell_idx,
                          const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                          int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                          float iso_value, int32_t dtype, const uint8_t* flags,
                          const int32_t* workspace, int64_t n_points, float* positions,
                          void* stream);

/* Replace `marching_cubes` (ash/src/grid.cu:606-946, pybind.cpp:31), which the
 * reference runs as four launches around two host read-backs, by two calls
 * around one read-back.  Tables and fields as for ash_isosurface_classify.
 *
 * classify: a listed cell takes part when it and the seven cells at its other
 * corners (entries 1..7 of the 8-entry neighbour tables) exist and weigh at
 * least weight_thr.  cases uint8[num_embeddings * cells_per_grid] receives its
 * case (bit c set when corner c is below iso_value; 0 = no surface) and
 * edge_slots uint32[num_embeddings * cells_per_grid] the flags of the +x/+y/+z
 * edges that carry a vertex; both need no initialisation, the entries of the
 * listed rows are cleared here, and every row that the neighbour table reaches
 * from a listed row must be listed too.  workspace (device int32, as many as
 * ash_marching_cubes_workspace_ints returns, no initialisation): [0] =
 * triangles, [1] = vertices, the rest is carried to extract.
 *
 * extract: after the caller has read workspace[0..1] and allocated positions
 * fp32[n_vertices, 3] (cell units) and triangles int32[n_triangles, 3] (vertex
 * ids, normals pointing from below iso_value to above it).  Vertices and
 * triangles come in the order of the listing, the same on every run.  May be
 * repeated after one classify.  At most 2^29 - 1 vertices. */
int64_t ash_marching_cubes_workspace_ints(int64_t num_grids, int64_t cells_per_grid);
int ash_marching_cubes_classify(const void* sdfs, const void* weights,
                                const int64_t* grid_indices,
                                const int64_t* lut_grid_nb2grid_idx,
                                const int32_t* cell_coords_table,
                                const int64_t* lut_cell_nb2cell_idx,
                                const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                                int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                                float iso_value, float weight_thr, int32_t dtype,
                                uint8_t* cases, uint32_t* edge_slots, int32_t* workspace,
                                void* stream);
int ash_marching_cubes_extract(const void* sdfs, const int64_t* grid_indices,
                               const int32_t* grid_coords_table,
                               const int64_t* lut_grid_nb2grid_idx,
                               const int32_t* cell_coords_table,
                               const int64_t* lut_cell_nb2cell_idx,
                               const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                               int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                               float iso_value, int32_t dtype, const uint8_t* cases,
                               uint32_t* edge_slots, int32_t* workspace, int64_t n_vertices,
                               int64_t n_triangles, float* positions, int32_t* triangles,
                               void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ASH_HIP_H_ */
