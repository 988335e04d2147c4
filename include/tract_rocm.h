/*
 * tract_rocm.h — C ABI of the MI355X (gfx950) KV-cache + attention path.
 *
 * This is the surface a `tract-rocm` runtime crate binds through FFI: plain
 * pointers, sizes and integer handles, no C++ or framework types.  Each entry point
 * names the interface of the tract tree it stands in for (paths relative to the
 * tract source tree, version 0.23.6-pre).
 *
 * Conventions
 *  - Every call returns 0 on success and 1 on failure; the message of the last
 *    failure on the calling thread is returned by trocm_last_error() and stays
 *    valid until the next failing call on that thread (same contract as tract's own
 *    C API, api/ffi/src/lib.rs:18-62).  Null pointers are reported, never
 *    dereferenced (api/ffi/src/lib.rs:83-92).
 *  - `stream` is a hipStream_t passed as void*.  Work is asynchronous and ordered by
 *    stream, one stream per host thread like cuda/src/context.rs:37-43.  NULL selects
 *    the library's own per-thread stream, never the legacy default stream.
 *  - Tensors are device pointers.  Shapes follow tract's attention layout
 *    [batch, heads, tokens, head_dim] with head_dim contiguous; rank-3 tensors are
 *    the heads == 1 case.  Strides are in elements unless the name says bytes.
 *  - All entry points may be called from several threads at once on distinct
 *    streams, caches and workspaces.
 */
#ifndef TRACT_ROCM_H
#define TRACT_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* Element / storage formats.  Q8_0 and Q4_0 are 32-element blocks along head_dim
 * with one f16 scale per block (canonical block bytes: linalg/src/frame/block_quant/
 * q4_0.rs:19-45, and q8_1.rs:20-48 without its `sum` field). */
typedef enum {
    TROCM_F32 = 0,
    TROCM_F16 = 1,
    TROCM_Q8_0 = 2,
    TROCM_Q4_0 = 3
} trocm_dtype;

/* ---- runtime ------------------------------------------------------------------ */

/* Select `device` and create the library context; idempotent.  Stands in for
 * cuda_context() (cuda/src/context.rs:28-35) / Runtime::check (core/src/runtime.rs:23-34). */
int trocm_init(int device);

/* Message of the last failing call on this thread (api/ffi/src/lib.rs:44-62). */
const char *trocm_last_error(void);

/* Device properties useful to a caller's scheduler: compute units, bytes of HBM. */
int trocm_device_info(int *compute_units, size_t *hbm_bytes, char *name, size_t name_len);

/* ---- device memory and streams: DeviceContext (gpu/src/device.rs:13-35) ---------- */

/* uninitialized_device_tensor (gpu/src/device.rs:15-19): 256-byte aligned device memory. */
int trocm_malloc(void **ptr, size_t bytes);
int trocm_free(void *ptr);
/* tensor_to_device (gpu/src/device.rs:14) / DeviceTensor::to_host (gpu/src/tensor/mod.rs:180-187).
 * Asynchronous on `stream`; the host buffer must stay alive until the stream is synchronised. */
int trocm_h2d(void *dst_device, const void *src_host, size_t bytes, void *stream);
int trocm_d2h(void *dst_host, const void *src_device, size_t bytes, void *stream);
int trocm_memset(void *dst_device, int byte_value, size_t bytes, void *stream);
int trocm_stream_create(void **stream);
int trocm_stream_destroy(void *stream);
/* DeviceContext::synchronize (gpu/src/device.rs:25) for one stream / for the device. */
int trocm_stream_sync(void *stream);
int trocm_device_sync(void);

/* Per-launch timing with event pairs, the device profiler's mechanism
 * (cuda/src/context.rs:363-453, cuda/src/kernels/launch_args.rs:77-90). */
int trocm_event_create(void **event);
int trocm_event_destroy(void *event);
int trocm_event_record(void *event, void *stream);
/* Waits for `stop`, then returns the time between the two events in milliseconds. */
int trocm_event_elapsed_ms(void *start, void *stop, float *ms);

/* DeviceContext::copy_nd (gpu/src/device.rs:26-35; CUDA: cuda/src/kernels/array/dispatch.rs:11-46):
 * strided N-d copy, rank 1..6, elem_size 1/2/4/8/16 bytes, strides in elements (may be
 * 0 for broadcast sources, never negative), byte offsets added to the base pointers. */
int trocm_copy_nd(void *dst, size_t dst_offset_bytes, const int64_t *dst_strides, const void *src,
                  size_t src_offset_bytes, const int64_t *src_strides, const int64_t *shape, int rank,
                  int elem_size, void *stream);

/* ---- in-place KV cache: InPlaceKvCache (transformers/src/ops/inplace_kv_cache.rs:28-114),
 *      replacing GpuDynKVCacheState::eval's reallocate-and-concat (gpu/src/ops/dyn_kv_cache.rs:58-113)
 *
 * One cache holds one tensor (K or V) of logical shape [batch, kv_heads, len, head_dim]
 * in a device buffer of `capacity` tokens.  Storage formats:
 *   F32/F16  [batch, kv_heads, capacity, head_dim]
 *   Q8_0     codes [batch, kv_heads, capacity, head_dim] bytes (code + 128) + scales [.., capacity, head_dim/32] f16
 *   Q4_0     codes [batch, kv_heads, capacity, head_dim/2] (16 canonical nibble bytes per block)
 *            + scales [.., capacity, head_dim/32] f16
 * The device layout of the quantised formats is private; trocm_kv_export() emits the
 * canonical block bytes (scale then codes, blocks row-major along head_dim). */
typedef struct trocm_kv_cache trocm_kv_cache;

/* A pool is ONE device allocation from which many caches take (and, on growth, exchange)
 * their planes: the arrangement for many independent sequences, each with its own
 * capacity-doubling cache.  It stands where DeviceMemoryPool (gpu/src/memory/pool.rs) stands
 * for per-run tensors, but for state that lives across runs.  Caches created in a pool
 * fail with a message when the pool is exhausted; destroy them before the pool. */
typedef struct trocm_kv_pool trocm_kv_pool;
int trocm_kv_pool_create(trocm_kv_pool **out, size_t bytes);
int trocm_kv_pool_destroy(trocm_kv_pool *pool);
int trocm_kv_pool_stats(trocm_kv_pool *pool, size_t *bytes_total, size_t *bytes_in_use, size_t *largest_free,
                        void **base);

/* InPlaceKvCache::new (:37-39).  Allocates nothing until the first append or reserve. */
int trocm_kv_cache_create(trocm_kv_cache **out, int storage_format, int64_t batch, int64_t kv_heads,
                          int64_t head_dim);
int trocm_kv_cache_create_in_pool(trocm_kv_cache **out, trocm_kv_pool *pool, int storage_format,
                                  int64_t batch, int64_t kv_heads, int64_t head_dim);
/* WindowKvCache::new (transformers/src/ops/window_kv_cache.rs:80-93): a fixed-capacity ring
 * buffer of `window` token slots for models trained with sliding-window attention.  Appends
 * overwrite the oldest slots once full (push, :111-143); len() <= window; the valid slots
 * are [0, len) in physical (rotated) order, which is all decode attention needs.  The
 * buffer is allocated at the first append; reserve and truncate are refused. */
int trocm_kv_cache_create_window(trocm_kv_cache **out, int storage_format, int64_t batch, int64_t kv_heads,
                                 int64_t head_dim, int64_t window);
/* window (0 for an ordinary cache) and the next write position. */
int trocm_kv_cache_window(const trocm_kv_cache *cache, int64_t *window, int64_t *cursor);
int trocm_kv_cache_destroy(trocm_kv_cache *cache);
/* len() / capacity() / reallocs() (:41-53). */
int trocm_kv_cache_len(const trocm_kv_cache *cache, int64_t *len);
int trocm_kv_cache_capacity(const trocm_kv_cache *cache, int64_t *capacity);
int trocm_kv_cache_reallocs(const trocm_kv_cache *cache, int64_t *reallocs);
/* Pre-allocate room for `capacity` tokens (no counterpart in the CPU op, whose Vec-like
 * growth starts from the first chunk; a device caller that knows its context budget
 * avoids every later reallocation).  Never shrinks; keeps the valid region. */
int trocm_kv_cache_reserve(trocm_kv_cache *cache, int64_t capacity, void *stream);
/* push (:55-85): append `n_new` tokens read from `src` ([batch, kv_heads, n_new, head_dim]
 * of src_dtype F32 or F16, element strides src_strides[4]; fused Move views are legal inputs
 * of the device cache op, cuda/src/rewrite_rules/fuse_axis_op.rs:13-27).  Growth rule (:61-80):
 * first chunk seeds capacity = n_new; else if len+n_new > capacity the buffer is replaced by
 * one of max(2*capacity, len+n_new) tokens holding the valid region.  A quantised cache
 * quantises on the way in; an F32/F16 cache requires src_dtype == storage_format. */
int trocm_kv_append(trocm_kv_cache *cache, const void *src, int src_dtype, const int64_t *src_strides,
                    int64_t n_new, void *stream);
/* The two pushes of InPlaceKvSdpaState::eval (inplace_kv_cache.rs:199-204) in one call and, for
 * F32/F16 caches with dense rows, one kernel launch: k_src and v_src share dtype and strides. */
int trocm_kv_append_pair(trocm_kv_cache *k_cache, trocm_kv_cache *v_cache, const void *k_src,
                         const void *v_src, int src_dtype, const int64_t *src_strides, int64_t n_new,
                         void *stream);
/* DynKeyValueCacheState::truncate (transformers/src/ops/dyn_kv_cache.rs:112-119): keep the first
 * `len` tokens (speculative-decoding rollback).  Fails on an empty cache like the reference. */
int trocm_kv_cache_truncate(trocm_kv_cache *cache, int64_t len);
/* valid_contiguous (:100-103) / OpState::save_to (:222-228): write the valid region, dense,
 * to `dst_device`: [batch, kv_heads, len, row_bytes] with row_bytes = trocm_kv_row_bytes(). */
int trocm_kv_export(const trocm_kv_cache *cache, void *dst_device, void *stream);
/* Bytes of one token of one head in the canonical export: head_dim*4, head_dim*2,
 * head_dim/32*34 or head_dim/32*18. */
int trocm_kv_row_bytes(const trocm_kv_cache *cache, size_t *bytes);
/* OpStateFreeze::freeze (:262-272): an independent deep copy (same len, capacity, reallocs). */
int trocm_kv_cache_clone(const trocm_kv_cache *cache, trocm_kv_cache **out, void *stream);
/* Raw view for kernels written against the cache: base pointers and the row pitch in tokens
 * (the planes are [batch, kv_heads, pitch, ...]; pitch >= capacity, large caches pad their rows
 * by 1/32 so that half-full power-of-two rows do not leave an address bit unused).
 * `scales` is NULL for F32/F16. */
int trocm_kv_cache_raw(const trocm_kv_cache *cache, void **data, void **scales, int64_t *pitch);

/* Append tokens given as canonical blocks in device memory, [batch, kv_heads, n_tokens,
 * head_dim/32 * block_bytes] (the layout trocm_kv_export writes): OpState::load_from
 * (dyn_kv_cache.rs:121-140) for a quantised cache without dequantising.  Quantised, ordinary
 * (not sliding-window) caches only; grows like an append. */
int trocm_kv_import_blocks(trocm_kv_cache *cache, const void *blocks_device, int64_t n_tokens, void *stream);

/* ---- NNEF tensor files (.dat), host memory only (nnef/src/tensors.rs) --------------------------
 * The 128-byte header (tensors.rs:10-25) for the tensors of this path.  `item` is a storage
 * format: TROCM_F32 / TROCM_F16 (vendor 0, item type 0; write_tensor :196-233), TROCM_Q4_0
 * (vendor 'TR', item type 0x3040, shape flattened to rank 2; write_block_quant_value :300-322)
 * or TROCM_Q8_0, written as tract's Q8_1 blocks of 36 bytes under item type 0x3081.
 * trocm_dat_header_read (read_tensor :62-95, read_block_quant_value :275-298) also accepts
 * item types 0x2040 (flag LEGACY_Q4_PACKING: convert the payload with
 * trocm_dat_q4_0_legacy_to_gguf, tensors.rs:250-273) and 0x3080; Q8 payloads are Q8_1 blocks
 * (flag Q8_1_BLOCKS: strip the sums with trocm_q8_1_to_q8_0 before trocm_kv_import_blocks). */
#define TROCM_DAT_LEGACY_Q4_PACKING 1
#define TROCM_DAT_Q8_1_BLOCKS 2
int trocm_dat_header_write(void *dst128, int item, int rank, const int64_t *dims, size_t data_bytes);
int trocm_dat_header_read(const void *src128, int *item, int *rank, int64_t *dims8, size_t *data_bytes, int *flags);
int trocm_dat_q4_0_legacy_to_gguf(void *blocks, size_t bytes);
int trocm_q8_1_to_q8_0(const void *src_36, void *dst_34, size_t n_blocks);
int trocm_q8_0_to_q8_1(const void *src_34, void *dst_36, size_t n_blocks);

/* ---- block quantisation as a tensor op: BlockQuant::{quant_f32,quant_f16,dequant_f32,dequant_f16}
 *      (linalg/src/frame/block_quant/mod.rs:48-108) ------------------------------------------- */

/* `n_elems` (multiple of 32) contiguous elements -> canonical blocks. */
int trocm_block_quant(int format, const void *src, int src_dtype, size_t n_elems, void *dst_blocks,
                      void *stream);
int trocm_block_dequant(int format, const void *src_blocks, size_t n_elems, void *dst, int dst_dtype,
                        void *stream);
/* BlockQuant::simulate_precision_loss (linalg/src/frame/block_quant/mod.rs:130-154; the matmul tests build
 * their expected values with it, test-rt/suite-unit/src/matmul_q40.rs:119-126): `n_elems` (multiple of 32)
 * contiguous elements of `dtype` (F32 / F16), blocked along the innermost axis, are quantised and dequantised
 * back into `dst` in one pass; `dst` may be `src`. */
int trocm_block_simulate_precision_loss(int format, const void *src, void *dst, int dtype, size_t n_elems,
                                        void *stream);

/* ---- Q4_0 weights x a few activation rows: the decode-time projections ------------------------
 *
 * The matrix-vector arm of GgmlGemm (cuda/src/kernels/matmul/mod.rs:575-627; taken for m <= 8,
 * :605-606; `dispatch_ggml_matvec_q40` :481-529): weights [batch, n, k] in Q4_0 blocks along k
 * (BlockQuantStorage rows, linalg/src/frame/block_quant/storage.rs:14-59), activations
 * [act_batch, m, k], output [act_batch, m, n] in the activations' type; act_batch must be a
 * multiple of the weights' batch (:488).  Result: the product with the dequantised weights, the
 * definition the reference's own test holds its kernel to (mod.rs:864-890).  More than 8 rows of f16
 * activations with k a multiple of 64 (weights held as tiles: more than 16 rows) take the matrix-matrix
 * arm (:607-610) on the matrix cores, with the weights dequantised to f16 as dequant_block_f16 stores them
 * (q4_0.rs:82-95); any other m > 8 runs as groups of 8 rows. */
typedef struct trocm_q4_weights trocm_q4_weights;

/* Device copy of `batch * n` rows of k/32 canonical 18-byte blocks (device pointer, row-major, no
 * padding; the reference pads rows to 512 elements for its kernel, cuda/src/utils.rs:252-280, which
 * this layout does not need).  k must be a multiple of 32 (utils.rs:253).  The copy is laid out for the
 * kernels, not for the caller: a matrix whose n is a multiple of 16 and whose k a multiple of 128 as tiles of
 * 16 rows x 128 features in the order the matrix instruction consumes them (one of up to 3072 rows -- the key
 * and value projections of a decoder with grouped heads -- keeps the planes beside the tiles, twice its bytes,
 * for calls with one or two activation rows), any other as a plane of codes and a plane of scales;
 * trocm_q4_0_weights_export returns the canonical blocks from either. */
int trocm_q4_0_weights_create(trocm_q4_weights **out, const void *blocks_device, int64_t batch, int64_t n,
                              int64_t k, void *stream);
int trocm_q4_0_weights_destroy(trocm_q4_weights *weights);
int trocm_q4_0_weights_shape(const trocm_q4_weights *weights, int64_t *batch, int64_t *n, int64_t *k);
/* The canonical blocks back (byte-identical to what was loaded). */
int trocm_q4_0_weights_export(const trocm_q4_weights *weights, void *dst_blocks_device, void *stream);
/* out[b, i, j] = sum_k act[b, i, k] * w[b / (act_batch / batch), j, k]; act and out dense, F32 or F16,
 * act 16-byte aligned.  One pass over the weights for the m <= 8 rows of a decode step (from about
 * 4 f16 rows on, and up to 16, on the matrix cores when k is a multiple of 128); a larger m of F16 rows
 * (k a multiple of 64) runs on a matrix-matrix kernel as the reference does (mod.rs:607-609), anything
 * else as groups of 8 rows, one pass each. */
int trocm_q4_0_matvec(const trocm_q4_weights *weights, const void *act, int act_dtype, int64_t act_batch,
                      int64_t m, void *out, void *stream);

/* ---- element-wise neighbours of the cache ------------------------------------------------- */

/* Planes that a growing cache or store has left behind are released behind an event by a later call of the library
 * (growth of a pooled cache, trocm_stream_sync, trocm_device_sync, a destroy, an allocation that fails at first).
 * A host that synchronises with its own HIP calls and never meets one of those can release them here: what the
 * device has finished with (wait == 0, never blocks on the stream) or everything (wait != 0).  No counterpart in
 * the reference, whose caches are freed by Rust's ownership (gpu/src/ops/dyn_kv_cache.rs:58-113). */
int trocm_release_unused(int wait);

/* A measurement aid with no counterpart in the reference: the floor under a launch of a given shape.
 * kind 0 launches a kernel that does nothing; kind 1 a kernel in which `workgroups` workgroups of `threads`
 * threads read `bytes` bytes at `src` once (non-temporal 128-bit loads) and write nothing (`sink`, 4 bytes of
 * device memory or NULL, is never written in practice).  Timed between two events on the stream, they say how
 * much of a short attention launch is the machine's launch and streaming time rather than the kernel's. */
int trocm_launch_floor(int kind, const void *src, size_t bytes, int workgroups, int threads, void *sink,
                       void *stream);

/* Cast between F32 and F16 (core `Cast` as the GPU backends run it,
 * cuda/src/kernels/array/cast.rs:21-47, :92): F32 -> F16 rounds to nearest even, F16 -> F32
 * is exact, same type copies.  n_elems dense elements. */
int trocm_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_elems, void *stream);

/* ApplyRope (transformers/src/ops/apply_rope.rs:169-176): out = x * cos + RotateHalf(x) * sin,
 * every product and the sum rounded to `dtype` like the CPU op.  Rank 2..4, inner dimension
 * even; strides in elements, NULL = dense.  cos and sin share `cos_sin_strides`, given for
 * the input's rank with 0 on broadcast axes (what compute_broadcast_strides produces in
 * cuda/src/kernels/nn/apply_rope.rs:75-81). */
int trocm_apply_rope(const void *input, const void *cos, const void *sin, void *out, int dtype, int rank,
                     const int64_t *shape, const int64_t *in_strides, const int64_t *cos_sin_strides,
                     const int64_t *out_strides, void *stream);

/* RotateHalf (transformers/src/ops/apply_rope.rs:58-76): out = concat(-x[.., h..], x[.., ..h])
 * along the innermost axis, h = half of it.  Rank 1..4. */
int trocm_rotate_half(const void *input, void *out, int dtype, int rank, const int64_t *shape,
                      const int64_t *in_strides, const int64_t *out_strides, void *stream);

/* ---- attention -------------------------------------------------------------------------- */

/* Scratch for split-K partial results and arrival counters.  The arena planner of the
 * device layer does not model scratch (gpu/src/memory/schema.rs:56-128), so the op state
 * owns one workspace and passes it to every call.  trocm_sdpa_workspace_init() must run
 * once on a new workspace (it zeroes the header area reserved for kernel-side counters);
 * kernels leave it ready for the next call.  Two calls that overlap in time must not share
 * a workspace; calls that follow each other on one stream may, dense and ragged in any order
 * (a ragged call keeps its launch plan in a second header area and refuses a workspace too
 * small to have one).  The size covers decode for (batch, q_heads, head_dim) and, for q_len > 1,
 * the partial results of a prefill whose key range is split over workgroups; a call made
 * with a smaller (or NULL) workspace still succeeds, with fewer splits. */
int trocm_sdpa_workspace_bytes(int64_t batch, int64_t q_heads, int64_t q_len, int64_t head_dim,
                               size_t *bytes);
int trocm_sdpa_workspace_init(void *workspace, size_t bytes, void *stream);

/* Sdpa (transformers/src/ops/sdpa.rs:83-89, semantics :131-227; CUDA dispatch
 * cuda/src/kernels/flash_attn.rs:82-189): out = softmax(q k^T * scale + mask) v.
 *   q, out : [batch, q_heads, q_len, head_dim] dense, dtype `dtype` (F32 or F16)
 *   k, v   : [batch, kv_heads, kv_len, head_dim] of the same dtype, element strides
 *            kv_strides[3] for batch, head, token (head_dim contiguous); q_heads must
 *            be a multiple of kv_heads, kv head = q head / group (sdpa.rs:156-164)
 *   mask   : optional additive [mask_batch, mask_heads, q_len, kv_len] dense, of `dtype`,
 *            mask_batch in {1, batch}, mask_heads in {1, q_heads} (the broadcast the CUDA
 *            dispatch expresses with zero strides, cuda/src/kernels/flash_attn.rs:138-143);
 *            must be NULL when causal (sdpa.rs:297-299).  Values may be finite minima
 *            (sdpa.rs:550-553) or -inf; a query row masked entirely with -inf yields zeros in every
 *            kernel: what the CPU op returns when its tile skip drops all of the row's key tiles
 *            (flash_sdpa.rs:267-274, :253; always so for q_len == 1), where its NaN for such a row
 *            inside a partly visible query tile (:309-316) is not reproduced.  The split-K decode and MFMA prefill kernels take the mask themselves; with
 *            q_len == 1 and mask_heads == 1 (a batch padded to its longest sequence,
 *            flash_sdpa.rs:261-268) the columns after the last one above -60000 weigh nothing and
 *            are not read.
 *   scale  : NaN selects the default 1/sqrt(head_dim) (sdpa.rs:177-181)
 *   causal : key j visible to query i iff j <= i + (kv_len - q_len) (flash_sdpa.rs:279-288) */
int trocm_sdpa(const void *q, const void *k, const void *v, const void *mask, void *out, int dtype,
               int64_t batch, int64_t q_heads, int64_t kv_heads, int64_t q_len, int64_t kv_len,
               int64_t head_dim, const int64_t *kv_strides, int64_t mask_batch, int64_t mask_heads,
               float scale, int causal, void *workspace, size_t workspace_bytes, void *stream);

/* The consumer half of InPlaceKvSdpaState::eval (inplace_kv_cache.rs:191-216): attention of
 * q over the valid [0..len] region of a K cache and a V cache, read in place (the device
 * twin of valid_view, :90-95), with fused dequantisation for Q8_0/Q4_0 caches.
 * q, out: [batch, q_heads, q_len, head_dim] dense of q_dtype (F32 or F16). */
int trocm_sdpa_cached(const void *q, int q_dtype, int64_t q_heads, int64_t q_len,
                      const trocm_kv_cache *k_cache, const trocm_kv_cache *v_cache, void *out,
                      float scale, int causal, void *workspace, size_t workspace_bytes, void *stream);

/* trocm_sdpa_cached for callers that cannot allocate device memory: tight serving loops, harnesses
 * that forbid hipMalloc.  (Recording it into a HIP graph is not tested, and of limited use: like every
 * attention entry point it passes the cache length to its kernels as an argument, so a replayed launch
 * would attend over the length it was recorded with.)  No counterpart in the reference.  Same
 * arguments, result and kernels as trocm_sdpa_cached, but the split-K scratch is a static device
 * array of TROCM_STATIC_SCRATCH_BYTES inside the library (held on the library's device until the
 * process ends) and the call reaches no hipMalloc, hipFree or other allocating routine.
 *   - `stream` must not be NULL (the library's per-thread stream is created on first use).
 *   - a shape whose trocm_sdpa_workspace_bytes(batch, q_heads, q_len, head_dim) exceeds
 *     TROCM_STATIC_SCRATCH_BYTES is refused with a message (decode: batch * q_heads <= 32768 at
 *     head_dim <= 128 fits; prefill: the split partials of q_len > 1 must fit).
 *   - every call shares the one array: calls that overlap in time on the device race on it;
 *     calls ordered by one stream, or by events, do not. */
#define TROCM_STATIC_SCRATCH_BYTES (24u << 20)
int trocm_sdpa_cached_noalloc(const void *q, int q_dtype, int64_t q_heads, int64_t q_len,
                              const trocm_kv_cache *k_cache, const trocm_kv_cache *v_cache, void *out,
                              float scale, int causal, void *stream);

/* InPlaceKvSdpaState::eval (inplace_kv_cache.rs:191-216) as one call: push k_new and v_new
 * ([batch, kv_heads, n_new, head_dim] of `dtype`, element strides kv_new_strides[4] or NULL for
 * dense) into the caches, then attend q ([batch, q_heads, n_new, head_dim] dense) over them. */
int trocm_inplace_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype,
                               int64_t q_heads, int64_t n_new, const int64_t *kv_new_strides,
                               trocm_kv_cache *k_cache, trocm_kv_cache *v_cache, void *out, float scale,
                               int causal, void *workspace, size_t workspace_bytes, void *stream);

/* ApplyRope (transformers/src/ops/apply_rope.rs:169-176) on q and k_new followed by InPlaceKvSdpaState::eval
 * (inplace_kv_cache.rs:191-216) as one call: the two ApplyRope nodes an exported decoder puts between its
 * projections and the cache (the pattern transformers/src/ops/sdpa.rs:453-458 looks through).  q, k_new, v_new and out
 * dense as in trocm_inplace_kv_sdpa_eval; cos and sin are [n_new, head_dim] rows of `dtype` per sequence,
 * `cos_sin_batch_stride` elements apart (0: one set of rows for every sequence); v_new is not rotated.  The appended
 * keys and the output are bit-identical to trocm_apply_rope on q and k_new followed by trocm_inplace_kv_sdpa_eval.
 * A single-token F16 step on an F16 cache with 2..16 query heads per kv head, or on a Q8_0 / Q4_0 cache (head_dim 128)
 * with 2..8, is one launch and touches no scratch (the key is rotated before it is quantised);
 * every other call rotates into `rot_scratch` (16-byte aligned), which must then hold
 * round_up(batch * q_heads * n_new * head_dim * elem, 256) + batch * kv_heads * n_new * head_dim * elem bytes
 * (a call that needs it and finds it too small fails before anything is changed). */
int trocm_inplace_kv_sdpa_eval_rope(const void *q, const void *k_new, const void *v_new, const void *cos,
                                    const void *sin, int64_t cos_sin_batch_stride, int dtype, int64_t q_heads,
                                    int64_t n_new, trocm_kv_cache *k_cache, trocm_kv_cache *v_cache, void *out,
                                    float scale, int causal, void *workspace, size_t workspace_bytes,
                                    void *rot_scratch, size_t rot_scratch_bytes, void *stream);

/* WindowKvSdpaState::eval (transformers/src/ops/window_kv_cache.rs:216-239): append K_new and
 * V_new to the two sliding-window caches, then attend Q to every valid slot without a causal
 * mask (the ring buffer is the window).  Arguments as trocm_inplace_kv_sdpa_eval.  A
 * single-token step on F32/F16 rings is one launch: the attention kernel stores the token at
 * the cursor. */
int trocm_window_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                              int64_t n_new, const int64_t *kv_new_strides, trocm_kv_cache *k_cache,
                              trocm_kv_cache *v_cache, void *out, float scale, void *workspace,
                              size_t workspace_bytes, void *stream);

/* Ragged multi-sequence decode: `n_seq` independent sequences, each with its own K and V
 * cache (batch == 1 each, same heads/head_dim/format) and its own length; one query token
 * per sequence.  q, out: [n_seq, q_heads, 1, head_dim].  The reference has no ragged batch:
 * its statement of the same result is a dense batch padded to the longest sequence with an
 * additive mask whose padded columns are <= -65504 (flash_sdpa.rs:261-268).  F16 and F32 caches,
 * and Q8_0 / Q4_0 caches with 1..32 query heads per kv head (head_dim 128, f16 queries), run as one launch (plus a merge launch
 * when a sequence is cut into more than 8 pieces); other cases as one call per sequence. */
int trocm_sdpa_decode_ragged(const void *q, int q_dtype, int64_t q_heads, int64_t n_seq,
                             trocm_kv_cache *const *k_caches, trocm_kv_cache *const *v_caches,
                             void *out, float scale, void *workspace, size_t workspace_bytes,
                             void *stream);

/* One decode step of a ragged batch as one call: append k_new[i], v_new[i] (dense
 * [n_seq, kv_heads, 1, head_dim] of `dtype`) to sequence i's caches, then attend q[i] over them.
 * Per sequence this is InPlaceKvSdpaState::eval (inplace_kv_cache.rs:191-216).  On F32/F16 caches
 * the attention kernel stores the new tokens itself: one launch (plus the split merge) per step;
 * on quantised caches one launch quantises every sequence's new token and a second attends. */
int trocm_inplace_kv_sdpa_eval_ragged(const void *q, const void *k_new, const void *v_new, int dtype,
                                      int64_t q_heads, int64_t n_seq, trocm_kv_cache *const *k_caches,
                                      trocm_kv_cache *const *v_caches, void *out, float scale,
                                      void *workspace, size_t workspace_bytes, void *stream);

/* The same step with ApplyRope (apply_rope.rs:169-176) on q and k_new folded in, as trocm_inplace_kv_sdpa_eval_rope does
 * for a dense batch: cos and sin are [n_seq, head_dim] rows of `dtype`, one per sequence (its position).  F16 steps over
 * F16 caches with 2..16 query heads per kv head, and over Q8_0 / Q4_0 caches with 2..8, rotate inside the attention
 * launch and touch no scratch; every other call rotates into `rot_scratch` (16-byte aligned,
 * round_up(n_seq * q_heads * head_dim * elem, 256) + n_seq * kv_heads * head_dim * elem bytes) first, and is refused
 * before anything changes when that is missing.  Bit-identical to trocm_apply_rope twice + the step above. */
int trocm_inplace_kv_sdpa_eval_ragged_rope(const void *q, const void *k_new, const void *v_new, const void *cos,
                                           const void *sin, int dtype, int64_t q_heads, int64_t n_seq,
                                           trocm_kv_cache *const *k_caches, trocm_kv_cache *const *v_caches, void *out,
                                           float scale, void *workspace, size_t workspace_bytes, void *rot_scratch,
                                           size_t rot_scratch_bytes, void *stream);

/* ---- KIVI-style affine quantised caches (the reference's own storage-quantised cache ops) ----------
 *
 * A different scheme from Q8_0 / Q4_0: u8 or u4 codes with f32 (lo, scale) parameters, Values per token,
 * Keys per channel.  One object holds one tensor [batch, heads, len, head_dim]; stored codes and
 * parameters are bit-identical to the CPU op's.
 *   TROCM_KIVI_PER_TOKEN        PerTokenStore (transformers/src/ops/quant_dyn_kv_cache.rs:97-151) and, with 8 bits
 *                               and no sink tokens, QuantValueCache (transformers/src/ops/kv_quant.rs:121-163)
 *   TROCM_KIVI_BLOCK_CHANNEL    BlockChannelStore (quant_dyn_kv_cache.rs:153-250): per-channel parameters frozen
 *                               per block of 32 tokens, the partial block kept in f32
 *   TROCM_KIVI_RUNNING_CHANNEL  QuantKeyCache (kv_quant.rs:171-236): running per-channel lo / scale, 8 bits; old
 *                               codes are read back with the current parameters, as the CPU op does
 * The first `sink_tokens` tokens stay in f32 (SINK_TOKENS = 4 in quant_dyn_kv_cache.rs:92; 0 in kv_quant.rs). */
typedef struct trocm_kivi_cache trocm_kivi_cache;
enum { TROCM_KIVI_PER_TOKEN = 0, TROCM_KIVI_BLOCK_CHANNEL = 1, TROCM_KIVI_RUNNING_CHANNEL = 2 };
enum { TROCM_KIVI_PART_SINK = 0, TROCM_KIVI_PART_CODES = 1, TROCM_KIVI_PART_LO = 2, TROCM_KIVI_PART_SCALE = 3,
       TROCM_KIVI_PART_RESIDUAL = 4 };

/* HeadCache::new for every (batch, head) (quant_dyn_kv_cache.rs:259-266, :401-406; kv_quant.rs:301-305).  bits is 4
 * or 8 (quant_dyn_kv_cache.rs:706).  Allocates at the first append. */
int trocm_kivi_cache_create(trocm_kivi_cache **out, int layout, int bits, int64_t sink_tokens, int64_t batch,
                            int64_t heads, int64_t head_dim);
int trocm_kivi_cache_destroy(trocm_kivi_cache *cache);
/* Back to the empty state a new session starts from (EvalOp::state, quant_dyn_kv_cache.rs:301-314), keeping the
 * device buffers. */
int trocm_kivi_cache_reset(trocm_kivi_cache *cache, void *stream);
int trocm_kivi_cache_len(const trocm_kivi_cache *cache, int64_t *len);
/* Tokens held as f32 sinks, as coded rows and in the partial key block; bytes of a coded row (row_bytes, :58-60). */
int trocm_kivi_cache_counts(const trocm_kivi_cache *cache, int64_t *n_sink, int64_t *n_rows, int64_t *n_res,
                            int64_t *row_bytes);
/* Resident bytes of the state: codes + 8 per parameter pair (memory_bytes, kv_quant.rs:160-162, :233-235) + the f32
 * sink and partial-block rows. */
int trocm_kivi_cache_memory_bytes(const trocm_kivi_cache *cache, size_t *bytes);
/* QuantizedDynKvCacheState::ingest (quant_dyn_kv_cache.rs:393-423): push every new token of `src`
 * ([batch, heads, n_new, head_dim] dense, F32 or F16; F16 is widened exactly like cast_to::<f32>, :487). */
int trocm_kivi_cache_append(trocm_kivi_cache *cache, const void *src, int src_dtype, int64_t n_new, void *stream);
/* QuantizedDynKvCacheState::dequantized + cast_to_dt (:426-449, :489): the whole cache as
 * [batch, heads, len, head_dim] dense of dst_dtype (F16 rounds to nearest even).  This is the op's output and
 * what save_to stores (:467-470). */
int trocm_kivi_cache_dequantize(const trocm_kivi_cache *cache, void *dst, int dst_dtype, void *stream);
/* One part of the raw state, dense per (batch, head): SINK [n_sink, head_dim] f32, CODES [n_rows, row_bytes],
 * LO / SCALE f32 ([n_rows] per token, [n_rows / 32, head_dim] per block and channel, [head_dim] running),
 * RESIDUAL [n_res, head_dim] f32.  `bytes` receives the size; a NULL dst only asks for it. */
int trocm_kivi_cache_export(const trocm_kivi_cache *cache, int part, void *dst_device, size_t *bytes, void *stream);
/* OpStateFreeze::freeze (quant_dyn_kv_cache.rs:510-524; kv_quant.rs:345-355): an independent deep copy. */
int trocm_kivi_cache_clone(const trocm_kivi_cache *cache, trocm_kivi_cache **out, void *stream);

/* QuantizedKvSdpaState::eval (kv_quant.rs:283-330): push k_new and v_new ([batch, kv_heads, n_new, head_dim] dense
 * of `dtype`) into a RUNNING_CHANNEL key store and a PER_TOKEN value store (8 bits, no sink tokens) and attend q
 * ([batch, q_heads, n_new, head_dim]) over every stored token WITHOUT a causal mask (:326).  One F16 query token at
 * head_dim 128 with up to 16 query heads per kv head attends straight over the codes (needs the workspace of
 * trocm_sdpa_workspace_bytes); every other case dequantises both stores into buffers they own (grown by doubling,
 * released again at the next step that does not need them) and runs trocm_sdpa over the copies. */
int trocm_quantized_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                                 int64_t n_new, trocm_kivi_cache *k_cache, trocm_kivi_cache *v_cache, void *out,
                                 float scale, void *workspace, size_t workspace_bytes, void *stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* TRACT_ROCM_H */
