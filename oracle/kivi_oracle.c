/*
 * CPU restatement of tract's KIVI-style affine KV-cache quantisers.  TEST INFRASTRUCTURE ONLY:
 * loaded by tests/, never by the product library.
 *
 * Follows, line by line:
 *   transformers/src/ops/kv_quant.rs:73-98        quant_dequant (any bit width, by row / by column)
 *   transformers/src/ops/kv_quant.rs:105-117      quant_token_to_u8 / dequant_u8
 *   transformers/src/ops/kv_quant.rs:121-163      QuantValueCache (per token, u8, no sink tokens)
 *   transformers/src/ops/kv_quant.rs:171-236      QuantKeyCache (running per-channel lo / scale)
 *   transformers/src/ops/quant_dyn_kv_cache.rs:52-90    max_code, row_bytes, pack_codes, unpack_code
 *   transformers/src/ops/quant_dyn_kv_cache.rs:92-151   SINK_TOKENS, PerTokenStore
 *   transformers/src/ops/quant_dyn_kv_cache.rs:153-250  KEY_BLOCK, BlockChannelStore
 *
 * Every float step is the reference's: f32 subtraction, IEEE division, f32::round (half away from
 * zero), clamp, saturating `as u8` (NaN -> 0); dequantisation is `lo + code * scale` with two
 * roundings (compiled with -ffp-contract=off).  f32::min / f32::max ignore a NaN operand of either kind
 * (rust_min / rust_max below; the C library's fminf / fmaxf answer NaN for a signalling one).  Parity unpinned: the sign of a zero `lo` (Rust leaves min(+0, -0) to the platform).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { KIVI_PER_TOKEN = 0, KIVI_BLOCK_CHANNEL = 1, KIVI_RUNNING_CHANNEL = 2 };
#define KEY_BLOCK 32 /* quant_dyn_kv_cache.rs:153 */

/* `x as u8` after `.round().clamp(0.0, lv)` (Rust: clamp keeps NaN, the cast turns it into 0). */
static uint8_t code_of(float x, float lo, float scale, float lv) {
    float q = roundf((x - lo) / scale);
    if (q != q) return 0;
    if (q < 0.0f) q = 0.0f;
    if (q > lv) q = lv;
    return (uint8_t)q;
}

/* f32::min / f32::max (core::f32): the other operand when one is NaN, quiet or signalling. */
static float rust_min(float a, float b) { return a != a ? b : (b != b ? a : (b < a ? b : a)); }
static float rust_max(float a, float b) { return a != a ? b : (b != b ? a : (b > a ? b : a)); }

/* kv_quant.rs:73-98 */
ORC_API void orc_kivi_quant_dequant(const float *x, size_t r, size_t c, unsigned bits, int by_row, float *out) {
    float levels = (float)((1u << bits) - 1u);
    size_t n_groups = by_row ? r : c, n_in = by_row ? c : r;
    for (size_t g = 0; g < n_groups; g++) {
        float lo = INFINITY, hi = -INFINITY;
        for (size_t k = 0; k < n_in; k++) {
            float v = by_row ? x[g * c + k] : x[k * c + g];
            lo = rust_min(lo, v);
            hi = rust_max(hi, v);
        }
        float scale = hi > lo ? (hi - lo) / levels : 1.0f;
        for (size_t k = 0; k < n_in; k++) {
            size_t at = by_row ? g * c + k : k * c + g;
            float q = roundf((x[at] - lo) / scale);
            /* f32::clamp keeps NaN */
            if (q == q) q = q < 0.0f ? 0.0f : (q > levels ? levels : q);
            out[at] = lo + q * scale;
        }
    }
}

typedef struct {
    int layout;
    size_t d, row_bytes, sink_tokens;
    unsigned bits;
    float *sink;
    size_t n_sink;
    uint8_t *packed;
    size_t n_rows, cap_rows; /* rows that hold codes */
    float *lo, *scale;       /* per token (n_rows), per block x channel (n_rows / 32 * d), or per channel (d) */
    size_t n_params, cap_params;
    float *residual;
    size_t n_res;
} orc_kivi;

static void reserve_rows(orc_kivi *s, size_t rows) {
    if (rows <= s->cap_rows) return;
    size_t cap = s->cap_rows ? s->cap_rows * 2 : 64;
    while (cap < rows) cap *= 2;
    s->packed = (uint8_t *)realloc(s->packed, cap * s->row_bytes);
    s->cap_rows = cap;
}
static void reserve_params(orc_kivi *s, size_t n) {
    if (n <= s->cap_params) return;
    size_t cap = s->cap_params ? s->cap_params * 2 : 64;
    while (cap < n) cap *= 2;
    s->lo = (float *)realloc(s->lo, cap * sizeof(float));
    s->scale = (float *)realloc(s->scale, cap * sizeof(float));
    s->cap_params = cap;
}

ORC_API void *orc_kivi_new(int layout, size_t d, unsigned bits, size_t sink_tokens) {
    orc_kivi *s = (orc_kivi *)calloc(1, sizeof(orc_kivi));
    s->layout = layout;
    s->d = d;
    s->bits = bits;
    s->row_bytes = (d * bits + 7) / 8; /* quant_dyn_kv_cache.rs:58-60 */
    s->sink_tokens = sink_tokens;
    s->sink = (float *)calloc(sink_tokens * d + 1, sizeof(float));
    s->residual = (float *)calloc(KEY_BLOCK * d, sizeof(float));
    if (layout == KIVI_RUNNING_CHANNEL) { /* kv_quant.rs:184-192 */
        reserve_params(s, d);
        s->n_params = d;
        for (size_t c = 0; c < d; c++) {
            s->lo[c] = INFINITY;
            s->scale[c] = 1.0f;
        }
    }
    return s;
}

ORC_API void orc_kivi_free(void *p) {
    orc_kivi *s = (orc_kivi *)p;
    if (!s) return;
    free(s->sink);
    free(s->packed);
    free(s->lo);
    free(s->scale);
    free(s->residual);
    free(s);
}

ORC_API void *orc_kivi_clone(const void *p) {
    const orc_kivi *s = (const orc_kivi *)p;
    orc_kivi *n = (orc_kivi *)malloc(sizeof(orc_kivi));
    *n = *s;
    n->sink = (float *)malloc((s->sink_tokens * s->d + 1) * sizeof(float));
    memcpy(n->sink, s->sink, (s->sink_tokens * s->d + 1) * sizeof(float));
    n->residual = (float *)malloc(KEY_BLOCK * s->d * sizeof(float));
    memcpy(n->residual, s->residual, KEY_BLOCK * s->d * sizeof(float));
    n->packed = (uint8_t *)malloc(s->cap_rows * s->row_bytes + 1);
    if (s->n_rows) memcpy(n->packed, s->packed, s->n_rows * s->row_bytes);
    n->lo = (float *)malloc((s->cap_params + 1) * sizeof(float));
    n->scale = (float *)malloc((s->cap_params + 1) * sizeof(float));
    if (s->n_params) {
        memcpy(n->lo, s->lo, s->n_params * sizeof(float));
        memcpy(n->scale, s->scale, s->n_params * sizeof(float));
    }
    return n;
}

/* quant_dyn_kv_cache.rs:64-77: bits = 8 one code per byte, bits = 4 even index -> low nibble */
static void pack_row(const uint8_t *codes, size_t d, unsigned bits, uint8_t *out) {
    if (bits == 8) {
        memcpy(out, codes, d);
    } else {
        for (size_t i = 0; i < d; i += 2) {
            uint8_t lo = codes[i] & 0x0F, hi = i + 1 < d ? (codes[i + 1] & 0x0F) : 0;
            out[i / 2] = (uint8_t)(lo | (hi << 4));
        }
    }
}
static uint8_t unpack_code(const uint8_t *row, size_t c, unsigned bits) { /* :80-90 */
    if (bits == 8) return row[c];
    uint8_t b = row[c >> 1];
    return (c & 1) == 0 ? (uint8_t)(b & 0x0F) : (uint8_t)(b >> 4);
}

/* quant_dyn_kv_cache.rs:165-199 */
static void finalize_block(orc_kivi *s) {
    size_t d = s->d;
    float lv = (float)((1u << s->bits) - 1u);
    reserve_params(s, s->n_params + d);
    float *lo = s->lo + s->n_params, *sc = s->scale + s->n_params;
    for (size_t c = 0; c < d; c++) {
        float l = INFINITY, h = -INFINITY;
        for (size_t t = 0; t < s->n_res; t++) {
            float v = s->residual[t * d + c];
            l = rust_min(l, v);
            h = rust_max(h, v);
        }
        lo[c] = l;
        sc[c] = h > l ? (h - l) / lv : 1.0f;
    }
    reserve_rows(s, s->n_rows + s->n_res);
    uint8_t *codes = (uint8_t *)malloc(d);
    for (size_t t = 0; t < s->n_res; t++) {
        for (size_t c = 0; c < d; c++) codes[c] = code_of(s->residual[t * d + c], lo[c], sc[c], lv);
        pack_row(codes, d, s->bits, s->packed + (s->n_rows + t) * s->row_bytes);
    }
    free(codes);
    s->n_rows += s->n_res;
    s->n_params += d;
    s->n_res = 0;
}

ORC_API void orc_kivi_push(void *p, const float *row) {
    orc_kivi *s = (orc_kivi *)p;
    size_t d = s->d;
    if (s->n_sink < s->sink_tokens) { /* quant_dyn_kv_cache.rs:118-122, :170-174 */
        memcpy(s->sink + s->n_sink * d, row, d * sizeof(float));
        s->n_sink++;
        return;
    }
    if (s->layout == KIVI_PER_TOKEN) { /* quant_dyn_kv_cache.rs:123-131 = kv_quant.rs:105-112 at 8 bits */
        float lv = (float)((1u << s->bits) - 1u);
        float lo = INFINITY, hi = -INFINITY;
        for (size_t c = 0; c < d; c++) {
            lo = rust_min(lo, row[c]);
            hi = rust_max(hi, row[c]);
        }
        float scale = hi > lo ? (hi - lo) / lv : 1.0f;
        uint8_t *codes = (uint8_t *)malloc(d);
        for (size_t c = 0; c < d; c++) codes[c] = code_of(row[c], lo, scale, lv);
        reserve_rows(s, s->n_rows + 1);
        pack_row(codes, d, s->bits, s->packed + s->n_rows * s->row_bytes);
        free(codes);
        reserve_params(s, s->n_params + 1);
        s->lo[s->n_params] = lo;
        s->scale[s->n_params] = scale;
        s->n_params++;
        s->n_rows++;
    } else if (s->layout == KIVI_BLOCK_CHANNEL) { /* quant_dyn_kv_cache.rs:175-180 */
        memcpy(s->residual + s->n_res * d, row, d * sizeof(float));
        s->n_res++;
        if (s->n_res == KEY_BLOCK) finalize_block(s);
    } else { /* kv_quant.rs:200-222 */
        for (size_t c = 0; c < d; c++) {
            float val = row[c];
            if (val < s->lo[c]) s->lo[c] = val;
            float range = val - s->lo[c];
            if (range > 0.0f) {
                float new_scale = (val - s->lo[c]) / 255.0f;
                if (new_scale > s->scale[c]) s->scale[c] = new_scale;
            }
        }
        reserve_rows(s, s->n_rows + 1);
        uint8_t *dst = s->packed + s->n_rows * s->row_bytes;
        for (size_t c = 0; c < d; c++) dst[c] = code_of(row[c], s->lo[c], s->scale[c], 255.0f);
        s->n_rows++;
    }
}

ORC_API size_t orc_kivi_len(const void *p) {
    const orc_kivi *s = (const orc_kivi *)p;
    return s->n_sink + s->n_rows + s->n_res;
}
ORC_API size_t orc_kivi_n_sink(const void *p) { return ((const orc_kivi *)p)->n_sink; }
ORC_API size_t orc_kivi_n_rows(const void *p) { return ((const orc_kivi *)p)->n_rows; }
ORC_API size_t orc_kivi_n_res(const void *p) { return ((const orc_kivi *)p)->n_res; }
ORC_API size_t orc_kivi_n_params(const void *p) { return ((const orc_kivi *)p)->n_params; }
ORC_API size_t orc_kivi_row_bytes(const void *p) { return ((const orc_kivi *)p)->row_bytes; }

/* Raw state, for byte comparisons: sink [n_sink, d] f32, packed [n_rows, row_bytes], lo / scale [n_params],
 * residual [n_res, d] f32.  Any destination may be NULL. */
ORC_API void orc_kivi_state(const void *p, float *sink, uint8_t *packed, float *lo, float *scale, float *residual) {
    const orc_kivi *s = (const orc_kivi *)p;
    if (sink) memcpy(sink, s->sink, s->n_sink * s->d * sizeof(float));
    if (packed && s->n_rows) memcpy(packed, s->packed, s->n_rows * s->row_bytes);
    if (lo && s->n_params) memcpy(lo, s->lo, s->n_params * sizeof(float));
    if (scale && s->n_params) memcpy(scale, s->scale, s->n_params * sizeof(float));
    if (residual) memcpy(residual, s->residual, s->n_res * s->d * sizeof(float));
}

/* dequant_all: quant_dyn_kv_cache.rs:132-150 (per token), :200-229 (block x channel),
 * kv_quant.rs:148-159 (per token, u8), :224-234 (running per channel: every stored code is read with the
 * CURRENT lo / scale of its channel).  out: [len, d]. */
ORC_API void orc_kivi_dequant_all(const void *p, float *out) {
    const orc_kivi *s = (const orc_kivi *)p;
    size_t d = s->d;
    memcpy(out, s->sink, s->n_sink * d * sizeof(float));
    float *o = out + s->n_sink * d;
    for (size_t t = 0; t < s->n_rows; t++) {
        const uint8_t *row = s->packed + t * s->row_bytes;
        for (size_t c = 0; c < d; c++) {
            float lo, sc;
            if (s->layout == KIVI_PER_TOKEN) {
                lo = s->lo[t];
                sc = s->scale[t];
            } else if (s->layout == KIVI_BLOCK_CHANNEL) {
                lo = s->lo[t / KEY_BLOCK * d + c];
                sc = s->scale[t / KEY_BLOCK * d + c];
            } else {
                lo = s->lo[c];
                sc = s->scale[c];
            }
            float prod = (float)unpack_code(row, c, s->bits) * sc;
            o[t * d + c] = lo + prod;
        }
    }
    memcpy(o + s->n_rows * d, s->residual, s->n_res * d * sizeof(float));
}

/* memory_bytes: kv_quant.rs:160-162 (packed + 8 per token), :233-235 (packed + 8 per channel). */
ORC_API size_t orc_kivi_memory_bytes(const void *p) {
    const orc_kivi *s = (const orc_kivi *)p;
    if (s->layout == KIVI_RUNNING_CHANNEL) return s->n_rows * s->row_bytes + s->d * 8;
    return s->n_rows * s->row_bytes + s->n_params * 8;
}
