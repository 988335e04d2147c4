// Internal declarations shared by the translation units of libtract_rocm.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/tract_rocm.h"

namespace trocm {

// ---- error convention: 0 = OK, 1 = KO + thread-local message --------------------------
int fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define TROCM_REQUIRE(cond, ...)                 \
    do {                                         \
        if (!(cond)) return ::trocm::fail(__VA_ARGS__); \
    } while (0)

#define TROCM_NOT_NULL(p) TROCM_REQUIRE((p) != nullptr, "unexpected null pointer argument: %s", #p)

#define TROCM_HIP(expr)                                                                   \
    do {                                                                                  \
        hipError_t e__ = (expr);                                                          \
        if (e__ != hipSuccess)                                                            \
            return ::trocm::fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__, __LINE__); \
    } while (0)

// Resolves the `void *stream` argument of the C ABI: NULL -> this thread's own stream.
int resolve_stream(void *stream, hipStream_t *out);
int ensure_init();
int num_compute_units();

static inline size_t elem_bytes(int dtype) { return dtype == TROCM_F32 ? 4 : dtype == TROCM_F16 ? 2 : 0; }
static inline bool is_quant(int fmt) { return fmt == TROCM_Q8_0 || fmt == TROCM_Q4_0; }
// Canonical bytes of one token row of one head.
static inline size_t canonical_row_bytes(int fmt, int64_t d) {
    switch (fmt) {
        case TROCM_F32: return (size_t)d * 4;
        case TROCM_F16: return (size_t)d * 2;
        case TROCM_Q8_0: return (size_t)d / 32 * 34;
        case TROCM_Q4_0: return (size_t)d / 32 * 18;
    }
    return 0;
}
// Bytes of one token row in the device code plane (F32/F16: the row itself).
static inline size_t device_row_bytes(int fmt, int64_t d) {
    switch (fmt) {
        case TROCM_F32: return (size_t)d * 4;
        case TROCM_F16: return (size_t)d * 2;
        case TROCM_Q8_0: return (size_t)d;
        case TROCM_Q4_0: return (size_t)d / 2;
    }
    return 0;
}

// ---- kernels' launchers (each in its own .hip file) ------------------------------------

// Strided N-d copy, strides in BYTES, rank <= 6.
struct CopyNd {
    int rank;
    int64_t shape[6];
    int64_t dst_stride[6];
    int64_t src_stride[6];
};
int launch_copy_nd(void *dst, const void *src, const CopyNd &desc, int elem_size, hipStream_t s);

// Two same-shaped appends (K and V) in one launch; rows dense, everything 16-byte aligned.
// Returns 2 when the shapes do not qualify (the caller then issues two copy_nd).
struct AppendPair {
    const void *src[2];
    void *dst[2];           // already offset to the first appended token
    int64_t B, H, S;
    int64_t row_bytes;
    int64_t src_stride[3];  // bytes: batch, head, token (same for both tensors)
    int64_t dst_stride[3];
};
int launch_append_pair(const AppendPair &a, hipStream_t s);
// Device memory that work queued on `s` may still read: released by a later call, once an event recorded on `s` now has
// completed (abi.hip).  reap_device_frees(wait) releases what has completed (wait: everything).
int defer_device_free(void *a, void *b, hipStream_t s);
void reap_device_frees(bool wait);
// empty kernel (kind 0) or read-only streaming kernel (kind 1) on a given launch shape
int launch_floor(int kind, const void *src, size_t bytes, int workgroups, int threads, void *sink, hipStream_t s);

// Quantise [rows, d] (row r of the source at src + b*ss[0] + h*ss[1] + t*ss[2] elements, element
// stride ss[3]) into the code/scale planes of a cache at token offset t0.
struct QuantAppend {
    int fmt, src_dtype;
    int64_t B, H, S, D;
    int64_t ss[4];          // source element strides
    int64_t cap, t0;        // destination capacity (tokens) and first token
    const void *src;
    void *codes, *scales;
};
int launch_quant_append(const QuantAppend &a, hipStream_t s);
// K and V of one shape and source type in one launch; returns 2 when they differ.
int launch_quant_append_pair(const QuantAppend &k, const QuantAppend &v, hipStream_t s);
// One new token for each of n_seq sequences (k_new / v_new dense [n_seq, H, 1, D], f16 or f32) quantised
// into the sequences' own K and V planes by one launch; `table` is in device memory.
struct QuantAppendSeq {
    void *k_codes, *k_scales, *v_codes, *v_scales;
    int64_t cap, t0;   // tokens between kv heads in the planes, and the token to write
};
int launch_quant_append_ragged(int fmt, int src_dtype, int64_t n_seq, int64_t H, int64_t D, const QuantAppendSeq *table,
                               const void *k_new, const void *v_new, hipStream_t s);
// A small host table (at most kWsPlanBytes) into device memory, ordered on the stream, by a kernel that reads
// pinned pages (a copy command between two kernels hands the stream to a DMA engine and back).
int upload_table(const void *src, size_t bytes, void *dst, hipStream_t s);
// Canonical export of the quantised planes: dst [B,H,len, D/32 * block_bytes].
int launch_quant_export(int fmt, int64_t B, int64_t H, int64_t len, int64_t cap, int64_t D,
                        const void *codes, const void *scales, void *dst, hipStream_t s);
// Canonical import: blocks [B,H,n, D/32 * block_bytes] into the planes at tokens [t0, t0 + n).
int launch_quant_import(int fmt, int64_t B, int64_t H, int64_t n, int64_t pitch, int64_t t0, int64_t D, const void *blocks,
                        void *codes, void *scales, hipStream_t s);
// Dequantise canonical blocks to a dense f32/f16 tensor.
int launch_block_quant(int fmt, const void *src, int src_dtype, size_t n_elems, void *dst, hipStream_t s);
int launch_block_dequant(int fmt, const void *blocks, size_t n_elems, void *dst, int dst_dtype, hipStream_t s);
// Quantise and dequantise in one pass (dst may be src): BlockQuant::simulate_precision_loss.
int launch_block_simulate(int fmt, const void *src, void *dst, int dtype, size_t n_elems, hipStream_t s);

// Element-wise neighbours of the cache: cast f32 <-> f16, RotateHalf, ApplyRope (rank <= 4, element
// strides, NULL = dense; cos/sin strides are 0 on broadcast axes).
int launch_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n, hipStream_t s);
int launch_apply_rope(const void *x, const void *cos, const void *sin, void *y, int dtype, int rank,
                      const int64_t *shape, const int64_t *in_strides, const int64_t *cs_strides,
                      const int64_t *out_strides, int rotate_only, hipStream_t s);

// Q4_0 weights (code plane [w_batch, n, k/2], scale plane [w_batch, n, k/32]) times m <= 8 activation
// rows: out[b, i, j] = sum_k act[b, i, k] * w[b * w_batch / act_batch, j, k]; act and out of act_dtype.
int launch_q4_0_matvec(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                       int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s);
// Q4_0 weights x 2..16 f16 activation rows on the matrix cores (q4_matvec_mfma.hip); 2 = not taken.
int launch_q4_0_matvec_mfma(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                            int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s);
// The same product for m > 8 rows of f16 activations on the matrix cores.  Returns 2 when not covered.
// tiled: `codes` are tiles of 16 rows x 128 features (q4_tiled.hip), `scales` is unused.
int launch_q4_0_matmul(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                       int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s, int tiled = 0);
// Q4_0 weights tiled by 16 rows x 128 features (n a multiple of 16, k of 128): the layout, its inverse, and the product
// with m rows of f16 or f32 activations (q4_tiled.hip).
bool q4_0_tiled_layout_fits(int64_t n, int64_t k);
size_t q4_0_tiled_bytes(int64_t rows, int64_t k);
int launch_q4_0_tiled_import(const void *blocks, void *tiles, int64_t rows, int64_t k, hipStream_t s);
int launch_q4_0_tiled_export(const void *tiles, void *blocks, int64_t rows, int64_t k, hipStream_t s);
int launch_q4_0_tiled_matvec(const void *tiles, int64_t w_batch, int64_t n, int64_t k, const void *act, int act_dtype,
                             int64_t act_batch, int64_t m, void *out, hipStream_t s);

// Attention.  One description for every kernel.
struct SdpaArgs {
    const void *q;
    void *out;
    int q_dtype;            // F32 / F16 (q and out)
    int kv_fmt;             // F32 / F16 / Q8_0 / Q4_0
    const void *k, *v;      // code planes (or plain tensors)
    const void *k_scales, *v_scales;
    // fused append (split-K decode of plain formats only): the new token's K and V rows, dense
    // [B, Hkv, 1, D]; they are token Sk-1, read from here and stored into the cache by the kernel
    const void *k_new, *v_new;
    int64_t new_pos;        // token index the fused new token is stored at; < 0 means Sk - 1 (ring buffers pass the cursor)
    int64_t B, Hq, Hkv, Sq, Sk, D;
    int64_t kv_stride_b, kv_stride_h, kv_stride_t;       // in ELEMENTS of the logical [.., D] tensor rows
    const void *mask;       // of q_dtype, [mask_b, mask_h, Sq, Sk]
    int64_t mask_b, mask_h;
    float scale;
    int causal;
    void *workspace;
    size_t workspace_bytes;
    // fused append with RoPE (f16 decode on the matrix cores only): q and k_new are rotated on the way in,
    // out = x * cos + RotateHalf(x) * sin with every product and the sum rounded to f16 like ApplyRope; rows of D
    // elements of q_dtype, one per batch entry `rope_stride_b` elements apart (0: one row for all)
    const void *rope_cos, *rope_sin;
    int64_t rope_stride_b;
};
int launch_sdpa_generic(const SdpaArgs &a, hipStream_t s);
// Split-K decode (Sq == 1).  Returns 2 when the shape is not covered by a fast kernel.
int launch_sdpa_decode(const SdpaArgs &a, hipStream_t s);
// Split-K decode for 2..32 query heads per kv head (f16): the heads are the rows of MFMA tiles.
// Returns 2 when not covered (masks, other types).
int launch_sdpa_decode_mfma(const SdpaArgs &a, hipStream_t s);
// Split-K decode over Q8_0 / Q4_0 caches with fused dequantisation.  Returns 2 when not covered.
int launch_sdpa_decode_quant(const SdpaArgs &a, hipStream_t s);
// Whether a step over a Q8_0 / Q4_0 cache with g_real query heads per kv head can rotate q and the new key (RoPE) inside the
// attention launch (sdpa_decode_mfma.hip).
bool decode_quant_rotates_in_kernel(int64_t g_real);
// Split-K decode straight over the affine u8 stores of QuantizedKvSdpa (kv_quant.rs:105-236): Keys coded per channel
// under one (lo, scale) per channel, Values per token.  f16 queries, head_dim 128, up to 16 query heads per kv head;
// returns 2 when not covered.
struct KiviSdpaArgs {
    const void *q;
    void *out;
    const uint8_t *k_codes, *v_codes;    // [B * Hkv, cap_rows, 128]
    int64_t k_cap_rows, v_cap_rows;
    const float *k_chan_scale;           // [B * Hkv, 128]
    const float *v_tok_scale, *v_tok_lo; // [B * Hkv, v_cap_rows]
    int64_t B, Hq, Hkv, T;
    float scale;
    void *workspace;
    size_t workspace_bytes;
};
int launch_sdpa_decode_kivi(const KiviSdpaArgs &a, hipStream_t s);
// MFMA prefill.  Returns 2 when the shape is not covered.
int launch_sdpa_prefill(const SdpaArgs &a, hipStream_t s);
// MFMA prefill for q_len >= 32: staggered waves, GQA heads sharing K/V tiles, key splits across
// workgroups (partials in the workspace after the counter area).  Returns 2 when not covered.
int launch_sdpa_prefill_pp(const SdpaArgs &a, hipStream_t s);
size_t prefill_workspace_bytes(int64_t B, int64_t Hq, int64_t Sq, int64_t D);

// Ragged decode: per-sequence descriptors live in pinned host memory owned by the library.
struct RaggedSeq {
    const void *k, *v, *k_scales, *v_scales;
    int64_t len, cap;
};
// k_new/v_new: optional fused append, dense [n_seq, Hkv, 1, D] (then seqs[i].len already counts
// the new token).  Returns 2 when a fused append was asked for but the fast kernel does not apply.
// rope_cos / rope_sin: with a fused append, rows [n_seq, D] of q_dtype by which q and k_new are rotated on the way in
// (2 when no kernel that does so covers the shape).
int launch_sdpa_decode_ragged(const void *q, void *out, int q_dtype, int kv_fmt, int64_t n_seq, int64_t Hq,
                              int64_t Hkv, int64_t D, const RaggedSeq *seqs, float scale, void *workspace,
                              size_t workspace_bytes, const void *k_new, const void *v_new, hipStream_t s,
                              const void *rope_cos = nullptr, const void *rope_sin = nullptr);

// Workspace layout: [arrival counters][partials ...]; a ragged launch keeps its plan (work items and
// per-sequence slot ranges) between the two, so that the counters stay zero for whichever launch comes next:
// [arrival counters][plan][partials ...].
constexpr size_t kWsCounterBytes = 64 * 1024;   // 16384 arrival counters
constexpr size_t kWsPlanBytes = 256 * 1024;     // about 3000 work items: the 2048 sequences a ragged launch takes, cut at most once each
size_t decode_workspace_bytes(int64_t B, int64_t Hq, int64_t D);

}  // namespace trocm
