/*
 * CPU ORACLE — TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the arithmetic of tract's CPU default runtime for the
 * KV-cache hot path.  Nothing here is part of the shipped product: only the test
 * suite, the smoke check and the benchmark's cpu_baseline leg may load this
 * library, and only as the checker.
 *
 * Each function cites the reference file:line whose behaviour it follows
 * (paths relative to the tract source tree, version 0.23.6-pre).
 *
 * Pin status (which independent facts each function was checked against lives in
 * tests/test_oracle_*.py):
 *   f16 conversions        pinned: exhaustive vs numpy.float16 (IEEE RNE)
 *   Q4_0 quant/dequant     pinned: reference known-answer round trips
 *                          (q4_0.rs:505-535,589-593,722-739) + hand-derived bytes
 *   Q8_1 / Q8_0 quant      pinned: hand-derived bytes from q8_1.rs:20-48 +
 *                          tolerance round trips (q8_1.rs:348-401)
 *   in-place cache / concat pinned: closed form == numpy.concatenate
 *                          (inplace_kv_cache.rs:366-418)
 *   flash SDPA / naive SDPA pinned (tolerance): reference golden io.npz files,
 *                          test-rt literal cases, f64 brute force, invariants.
 *                          Bit-level f32 parity of attention is unpinned by design:
 *                          the reference's dot products run in the third-party
 *                          crate matrixmultiply 0.3.10 whose summation order is not
 *                          part of the reference tree.
 *
 *   window (ring) cache     pinned: the reference's unit tests (window_kv_cache.rs:342-374:
 *                          last-w-as-a-set, chunk larger than the window), hand-derived
 *                          slot layouts for the wrap-around case, windowed attention ==
 *                          attention over the last w tokens (:407-466)
 *   RotateHalf / ApplyRope  pinned: RotateHalf twice == negation (the reference's own unit
 *                          test, apply_rope.rs:257-277), an independent numpy
 *                          concatenate form, the rotation closed forms (norm of each
 *                          pair kept, angles add); f16 arithmetic is the `half` crate's
 *                          (operate in f32, round to f16 after every operation)
 *   StreamedSdpaOp          pinned (tolerance): f64 brute force with its own mask rules (top-left causal,
 *                          rank-2 mask that overrides the causal flag), independence of block_k, rows that
 *                          see nothing are zero; equals the flash path where their rules coincide
 *   Q4_0 matrix-vector      pinned (tolerance): == numpy's product with the (pinned) dequantised
 *                          weights in f64, a hand-built block whose dot product is known in
 *                          closed form, linearity in the activations; exact f32 bits unpinned
 *                          (summation order of the CPU matrix product)
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off (Rust never contracts a*b+c).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* IEEE binary16 <-> binary32, round-to-nearest-even (crate `half` 2.7.1       */
/* f16::from_f32 / f16::to_f32 semantics; Cargo.lock:1672).                     */
/* ------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

ORC_API uint16_t orc_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        /* quiet the nan, keep top mantissa bits */
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
    if (e <= 0) {
        /* subnormal half or zero */
        if (e < -10) return (uint16_t)sign; /* too small: rounds to zero */
        man |= 0x800000u;                   /* implicit bit */
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man); /* carry into exponent is correct */
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry to inf */
    return (uint16_t)(sign | half);
}

ORC_API float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: normalise */
        int e = -1;
        do {
            e++;
            man <<= 1;
        } while (!(man & 0x400u));
        man &= 0x3ffu;
        return bits_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
    }
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp - 15 + 127) << 23) | (man << 13));
}

ORC_API void orc_f32_to_f16_n(const float *src, uint16_t *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_f16(src[i]);
}
ORC_API void orc_f16_to_f32_n(const uint16_t *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_f16_to_f32(src[i]);
}

/* Rust `f32 as i8`: truncate toward zero, saturate, NaN -> 0. */
static inline int8_t rust_f32_as_i8(float x) {
    if (x != x) return 0;
    if (x <= -128.0f) return -128;
    if (x >= 127.0f) return 127;
    return (int8_t)x; /* C truncation toward zero, in range */
}

/* ------------------------------------------------------------------------- */
/* Q4_0: 32 elements -> f16 scale + 16 nibble bytes = 18 B                      */
/* linalg/src/frame/block_quant/q4_0.rs:19-45 (quant_block), :82-95 (dequant).  */
/* Nibble order: helpers.rs:41-73 — first write = low nibble.                   */
/* ------------------------------------------------------------------------- */

#define QK 32

ORC_API void orc_q4_0_quant_block_f32(const float *block, uint8_t *quant) {
    /* q4_0.rs:27-34: signed value of the first element with strictly largest |v| */
    float amax = 0.0f, max = 0.0f;
    for (int i = 0; i < QK; i++) {
        float a = fabsf(block[i]);
        if (amax < a) {
            amax = a;
            max = block[i];
        }
    }
    float scale = max / -8.0f;                              /* q4_0.rs:35 */
    float r_scale = (scale == 0.0f) ? 0.0f : 1.0f / scale;  /* q4_0.rs:36 */
    uint16_t d = orc_f32_to_f16(scale);                      /* q4_0.rs:37 */
    quant[0] = (uint8_t)(d & 0xff);
    quant[1] = (uint8_t)(d >> 8);
    /* q4_0.rs:39-44: idx -> ggml_idx = 16*(idx%2) + idx/2, two nibbles per byte */
    for (int j = 0; j < QK / 2; j++) {
        float lo_f = block[j] * r_scale;
        lo_f = lo_f + 8.5f;
        float hi_f = block[j + QK / 2] * r_scale;
        hi_f = hi_f + 8.5f;
        int8_t lo = rust_f32_as_i8(lo_f);
        int8_t hi = rust_f32_as_i8(hi_f);
        if (lo > 15) lo = 15;
        if (hi > 15) hi = 15;
        /* helpers.rs:62-68: first as u8 | (second as u8) << 4, in u8 arithmetic */
        quant[2 + j] = (uint8_t)((uint8_t)lo | (uint8_t)((uint8_t)hi << 4));
    }
}

ORC_API void orc_q4_0_quant_block_f16(const uint16_t *block, uint8_t *quant) {
    /* q4_0.rs:19-45 with T = f16: comparisons and abs on f16 are exact images of
     * the widened f32 values; all arithmetic is on f32::from(v). */
    float tmp[QK];
    for (int i = 0; i < QK; i++) tmp[i] = orc_f16_to_f32(block[i]);
    orc_q4_0_quant_block_f32(tmp, quant);
}

ORC_API void orc_q4_0_dequant_block_f32(const uint8_t *quant, float *block) {
    float d = orc_f16_to_f32((uint16_t)(quant[0] | (quant[1] << 8)));
    for (int j = 0; j < QK / 2; j++) {
        int lo = quant[2 + j] & 0x0f, hi = quant[2 + j] >> 4;
        block[j] = (float)(lo - 8) * d; /* q4_0.rs:93 */
        block[j + QK / 2] = (float)(hi - 8) * d;
    }
}

ORC_API void orc_q4_0_dequant_block_f16(const uint8_t *quant, uint16_t *block) {
    /* T = f16: (nibble-8) as f16 (exact) times d, `half` multiplies in f32 then
     * rounds the product to f16 (RNE). */
    float d = orc_f16_to_f32((uint16_t)(quant[0] | (quant[1] << 8)));
    for (int j = 0; j < QK / 2; j++) {
        int lo = quant[2 + j] & 0x0f, hi = quant[2 + j] >> 4;
        block[j] = orc_f32_to_f16((float)(lo - 8) * d);
        block[j + QK / 2] = orc_f32_to_f16((float)(hi - 8) * d);
    }
}

/* ------------------------------------------------------------------------- */
/* Q8_1: 32 elements -> f16 scale, f16 sum, 32 x i8 = 36 B  (q8_1.rs:20-48)     */
/* Q8_0 = the same block without the `sum` field = 34 B (d, then 32 codes).     */
/* ------------------------------------------------------------------------- */

static void q8_codes_f32(const float *block, float *scale_out, int8_t *codes) {
    float amax = 0.0f, max = 0.0f;
    for (int i = 0; i < QK; i++) { /* q8_1.rs:30-37 */
        float a = fabsf(block[i]);
        if (amax < a) {
            amax = a;
            max = block[i];
        }
    }
    float scale = max / 127.0f;                             /* q8_1.rs:39 */
    float r_scale = (scale == 0.0f) ? 0.0f : 1.0f / scale;  /* q8_1.rs:40 */
    *scale_out = scale;
    for (int i = 0; i < QK; i++) {
        float p = block[i] * r_scale;
        codes[i] = rust_f32_as_i8(roundf(p)); /* q8_1.rs:45: round half away from zero */
    }
}

ORC_API void orc_q8_0_quant_block_f32(const float *block, uint8_t *quant) {
    float scale;
    q8_codes_f32(block, &scale, (int8_t *)(quant + 2));
    uint16_t d = orc_f32_to_f16(scale);
    quant[0] = (uint8_t)(d & 0xff);
    quant[1] = (uint8_t)(d >> 8);
}

ORC_API void orc_q8_0_quant_block_f16(const uint16_t *block, uint8_t *quant) {
    float tmp[QK];
    for (int i = 0; i < QK; i++) tmp[i] = orc_f16_to_f32(block[i]);
    orc_q8_0_quant_block_f32(tmp, quant);
}

ORC_API void orc_q8_1_quant_block_f32(const float *block, uint8_t *quant) {
    float scale;
    q8_codes_f32(block, &scale, (int8_t *)(quant + 4));
    float sum = 0.0f; /* q8_1.rs:36: sum += *v in T = f32, sequential */
    for (int i = 0; i < QK; i++) sum += block[i];
    uint16_t d = orc_f32_to_f16(scale), s = orc_f32_to_f16(sum);
    quant[0] = (uint8_t)(d & 0xff);
    quant[1] = (uint8_t)(d >> 8);
    quant[2] = (uint8_t)(s & 0xff);
    quant[3] = (uint8_t)(s >> 8);
}

ORC_API void orc_q8_1_quant_block_f16(const uint16_t *block, uint8_t *quant) {
    float tmp[QK];
    for (int i = 0; i < QK; i++) tmp[i] = orc_f16_to_f32(block[i]);
    float scale;
    q8_codes_f32(tmp, &scale, (int8_t *)(quant + 4));
    /* q8_1.rs:36 with T = f16: each `+=` is an f16 add (f32 add, rounded to f16). */
    uint16_t sum = 0;
    for (int i = 0; i < QK; i++) sum = orc_f32_to_f16(orc_f16_to_f32(sum) + tmp[i]);
    uint16_t d = orc_f32_to_f16(scale);
    quant[0] = (uint8_t)(d & 0xff);
    quant[1] = (uint8_t)(d >> 8);
    quant[2] = (uint8_t)(sum & 0xff);
    quant[3] = (uint8_t)(sum >> 8);
}

static void q8_dequant_f32(const uint8_t *dptr, const int8_t *codes, float *block) {
    float d = orc_f16_to_f32((uint16_t)(dptr[0] | (dptr[1] << 8)));
    for (int i = 0; i < QK; i++) block[i] = (float)codes[i] * d; /* q8_1.rs:60-62 */
}
static void q8_dequant_f16(const uint8_t *dptr, const int8_t *codes, uint16_t *block) {
    float d = orc_f16_to_f32((uint16_t)(dptr[0] | (dptr[1] << 8)));
    for (int i = 0; i < QK; i++) block[i] = orc_f32_to_f16((float)codes[i] * d);
}
ORC_API void orc_q8_0_dequant_block_f32(const uint8_t *q, float *b) {
    q8_dequant_f32(q, (const int8_t *)(q + 2), b);
}
ORC_API void orc_q8_0_dequant_block_f16(const uint8_t *q, uint16_t *b) {
    q8_dequant_f16(q, (const int8_t *)(q + 2), b);
}
ORC_API void orc_q8_1_dequant_block_f32(const uint8_t *q, float *b) {
    q8_dequant_f32(q, (const int8_t *)(q + 4), b);
}
ORC_API void orc_q8_1_dequant_block_f16(const uint8_t *q, uint16_t *b) {
    q8_dequant_f16(q, (const int8_t *)(q + 4), b);
}

/* Format ids shared with the tests: 2 = Q8_0, 3 = Q4_0, 4 = Q8_1. */
ORC_API size_t orc_block_bytes(int fmt) { return fmt == 3 ? 18 : fmt == 2 ? 34 : fmt == 4 ? 36 : 0; }

/* BlockQuant::quant_f32 / quant_f16 (block_quant/mod.rs:48-76): a row-major
 * sequence of blocks along the last axis; src_f16 selects the input type. */
ORC_API int orc_quant(int fmt, int src_f16, const void *src, size_t n_elems, uint8_t *dst) {
    size_t bb = orc_block_bytes(fmt);
    if (!bb || n_elems % QK) return 1;
    for (size_t b = 0; b < n_elems / QK; b++) {
        uint8_t *q = dst + b * bb;
        if (src_f16) {
            const uint16_t *s = (const uint16_t *)src + b * QK;
            if (fmt == 3) orc_q4_0_quant_block_f16(s, q);
            else if (fmt == 2) orc_q8_0_quant_block_f16(s, q);
            else orc_q8_1_quant_block_f16(s, q);
        } else {
            const float *s = (const float *)src + b * QK;
            if (fmt == 3) orc_q4_0_quant_block_f32(s, q);
            else if (fmt == 2) orc_q8_0_quant_block_f32(s, q);
            else orc_q8_1_quant_block_f32(s, q);
        }
    }
    return 0;
}

/* BlockQuant::dequant_f32 / dequant_f16 (block_quant/mod.rs:78-108). */
ORC_API int orc_dequant(int fmt, int dst_f16, const uint8_t *src, size_t n_elems, void *dst) {
    size_t bb = orc_block_bytes(fmt);
    if (!bb || n_elems % QK) return 1;
    for (size_t b = 0; b < n_elems / QK; b++) {
        const uint8_t *q = src + b * bb;
        if (dst_f16) {
            uint16_t *o = (uint16_t *)dst + b * QK;
            if (fmt == 3) orc_q4_0_dequant_block_f16(q, o);
            else if (fmt == 2) orc_q8_0_dequant_block_f16(q, o);
            else orc_q8_1_dequant_block_f16(q, o);
        } else {
            float *o = (float *)dst + b * QK;
            if (fmt == 3) orc_q4_0_dequant_block_f32(q, o);
            else if (fmt == 2) orc_q8_0_dequant_block_f32(q, o);
            else orc_q8_1_dequant_block_f32(q, o);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Q4_0 weights x activations: out[b, i, j] = sum_k act[b, i, k] * w[b / ratio, j, k], the product the */
/* reference holds its GPU kernel to (cuda/src/kernels/matmul/mod.rs:864-890): the weights pass         */
/* through Q4_0.simulate_precision_loss (quantise + dequantise in the activations' type,               */
/* block_quant/mod.rs:110-155) and then a plain matrix product in that type.  Here the blocks are       */
/* given; each is dequantised in the activations' type (f16: rounded to f16, q4_0.rs:82-95) and the     */
/* dot product accumulates in f32 in k order (the exact f32 bits of the CPU product depend on the      */
/* matrix-multiply kernel's summation order and are not pinned; callers compare within a tolerance).   */
/* ------------------------------------------------------------------------- */
ORC_API int orc_q4_0_matvec(const uint8_t *blocks, size_t w_batch, size_t n, size_t k, const void *act, int f16,
                            size_t act_batch, size_t m, void *out) {
    if (k % QK || w_batch == 0 || act_batch % w_batch) return 1;
    const size_t ratio = act_batch / w_batch, nb = k / QK, rb = nb * 18;
    long long total = (long long)act_batch * (long long)n;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (long long bj = 0; bj < total; bj++) {
        const size_t b = (size_t)bj / n, j = (size_t)bj % n;
        const uint8_t *row = blocks + ((b / ratio) * n + j) * rb;
        for (size_t i = 0; i < m; i++) {
            float acc = 0.0f;
            for (size_t blk = 0; blk < nb; blk++) {
                float w[QK];
                if (f16) {
                    uint16_t h[QK];
                    orc_q4_0_dequant_block_f16(row + blk * 18, h);
                    for (int e = 0; e < QK; e++) w[e] = orc_f16_to_f32(h[e]);
                } else {
                    orc_q4_0_dequant_block_f32(row + blk * 18, w);
                }
                for (int e = 0; e < QK; e++) {
                    const size_t kk = blk * QK + e;
                    const float x = f16 ? orc_f16_to_f32(((const uint16_t *)act)[(b * m + i) * k + kk])
                                        : ((const float *)act)[(b * m + i) * k + kk];
                    acc += w[e] * x;
                }
            }
            if (f16) ((uint16_t *)out)[(b * m + i) * n + j] = orc_f32_to_f16(acc);
            else ((float *)out)[(b * m + i) * n + j] = acc;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* KV cache, host side.  A tensor [outer, len, inner] of `elem` bytes, sequence */
/* axis in the middle (outer = product of dims before the axis, inner = product */
/* after).                                                                      */
/* ------------------------------------------------------------------------- */

typedef struct {
    size_t outer, inner_bytes; /* bytes of one [inner] row */
    size_t len, cap, reallocs;
    uint8_t *buf; /* [outer, cap, inner_bytes] */
} orc_kv_cache;

ORC_API orc_kv_cache *orc_kv_new(size_t outer, size_t inner_bytes) {
    orc_kv_cache *c = (orc_kv_cache *)calloc(1, sizeof(*c));
    c->outer = outer;
    c->inner_bytes = inner_bytes;
    return c;
}
ORC_API void orc_kv_free(orc_kv_cache *c) {
    if (c) {
        free(c->buf);
        free(c);
    }
}
ORC_API size_t orc_kv_len(const orc_kv_cache *c) { return c->len; }
ORC_API size_t orc_kv_capacity(const orc_kv_cache *c) { return c->cap; }
ORC_API size_t orc_kv_reallocs(const orc_kv_cache *c) { return c->reallocs; }
ORC_API const uint8_t *orc_kv_buffer(const orc_kv_cache *c) { return c->buf; }

/* Tensor::assign_slice along the axis (data/src/tensor.rs:833-935): copy
 * src[:, s0:s0+n, :] (capacity src_cap) into dst[:, d0:d0+n, :] (capacity dst_cap). */
static void assign_slice(uint8_t *dst, size_t dst_cap, size_t d0, const uint8_t *src, size_t src_cap,
                         size_t s0, size_t n, size_t outer, size_t inner_bytes) {
    for (size_t o = 0; o < outer; o++)
        memcpy(dst + (o * dst_cap + d0) * inner_bytes, src + (o * src_cap + s0) * inner_bytes,
               n * inner_bytes);
}

/* InPlaceKvCache::push (transformers/src/ops/inplace_kv_cache.rs:55-85) with
 * grow (:106-113).  `input` is a dense [outer, n_new, inner]. */
ORC_API int orc_kv_push(orc_kv_cache *c, const uint8_t *input, size_t n_new) {
    if (n_new == 0) return 0; /* :57-59 */
    if (!c->buf) {            /* :61-66: seed, capacity = first chunk length */
        c->buf = (uint8_t *)malloc(c->outer * n_new * c->inner_bytes);
        if (!c->buf) return 1;
        memcpy(c->buf, input, c->outer * n_new * c->inner_bytes);
        c->cap = n_new;
        c->len = n_new;
        return 0;
    }
    if (c->len + n_new <= c->cap) { /* :70-73 */
        assign_slice(c->buf, c->cap, c->len, input, n_new, 0, n_new, c->outer, c->inner_bytes);
        c->len += n_new;
        return 0;
    }
    /* :75-80 */
    size_t new_cap = c->cap * 2 > c->len + n_new ? c->cap * 2 : c->len + n_new;
    uint8_t *grown = (uint8_t *)malloc(c->outer * new_cap * c->inner_bytes);
    if (!grown) return 1;
    assign_slice(grown, new_cap, 0, c->buf, c->cap, 0, c->len, c->outer, c->inner_bytes);
    assign_slice(grown, new_cap, c->len, input, n_new, 0, n_new, c->outer, c->inner_bytes);
    free(c->buf);
    c->buf = grown;
    c->cap = new_cap;
    c->len += n_new;
    c->reallocs += 1;
    return 0;
}

/* InPlaceKvCache::valid_contiguous (:100-103): dense copy of [0..len]. */
ORC_API void orc_kv_valid_contiguous(const orc_kv_cache *c, uint8_t *dst) {
    if (c->len) assign_slice(dst, c->len, 0, c->buf, c->cap, 0, c->len, c->outer, c->inner_bytes);
}

/* DynKeyValueCacheState::eval (transformers/src/ops/dyn_kv_cache.rs:158-174):
 * TypedConcat -> Tensor::stack_tensors (data/src/tensor.rs:354-): a fresh
 * allocation holding the whole past followed by the new chunk.  Returns the new
 * dense [outer, past+n_new, inner] buffer (caller frees with orc_free). */
ORC_API uint8_t *orc_concat_append(const uint8_t *past, size_t past_len, const uint8_t *input,
                                   size_t n_new, size_t outer, size_t inner_bytes) {
    size_t total = past_len + n_new;
    uint8_t *out = (uint8_t *)malloc(outer * total * inner_bytes + 1);
    if (!out) return NULL;
    if (past_len) assign_slice(out, total, 0, past, past_len, 0, past_len, outer, inner_bytes);
    if (n_new) assign_slice(out, total, past_len, input, n_new, 0, n_new, outer, inner_bytes);
    return out;
}
ORC_API void orc_free(void *p) { free(p); }

/* ------------------------------------------------------------------------- */
/* Attention.                                                                   */
/* ------------------------------------------------------------------------- */

/* FlashSdpaOp::attend_one_head (transformers/src/ops/flash_sdpa.rs:239-341).
 * q: [q_len, d] contiguous rows; k, v: rows of d contiguous floats, consecutive
 * tokens `kv_row_stride` floats apart (so a view into a capacity buffer works,
 * like InPlaceKvCache::valid_view); mask: optional [q_len, kv_len] slice with the
 * given row stride; out: [q_len, d]. */
static void attend_one_head(const float *q, const float *k, const float *v, size_t kv_row_stride,
                            const float *mask, size_t mask_row_stride, size_t q_len, size_t kv_len,
                            size_t d, int causal, float scale, float *out) {
    enum { BKV = 32, BQ = 32 }; /* :248-249 */
    float *l = (float *)malloc(q_len * sizeof(float));
    float *m = (float *)malloc(q_len * sizeof(float));
    float *s = (float *)malloc(BQ * BKV * sizeof(float));
    float *sv = (float *)malloc(BQ * d * sizeof(float));
    for (size_t i = 0; i < q_len; i++) {
        l[i] = 0.0f;
        m[i] = -INFINITY;
    }
    memset(out, 0, q_len * d * sizeof(float));
    size_t n_kb = (kv_len + BKV - 1) / BKV, n_qb = (q_len + BQ - 1) / BQ;
    for (size_t kb = 0; kb < n_kb; kb++) {     /* :257 kv-outer */
        for (size_t qb = 0; qb < n_qb; qb++) { /* :258 q-inner */
            size_t kv0 = kb * BKV, kv1 = kv0 + BKV < kv_len ? kv0 + BKV : kv_len;
            size_t q0 = qb * BQ, q1 = q0 + BQ < q_len ? q0 + BQ : q_len;
            size_t nq = q1 - q0, nk = kv1 - kv0;
            if (mask) { /* :261-268: skip a tile whose mask is entirely < -65503 */
                int all = 1;
                for (size_t i = 0; i < nq && all; i++)
                    for (size_t j = 0; j < nk; j++)
                        if (!(mask[(q0 + i) * mask_row_stride + kv0 + j] < -65503.0f)) {
                            all = 0;
                            break;
                        }
                if (all) continue;
            }
            /* :276  s = (Qb . Kb^T) * scale */
            for (size_t i = 0; i < nq; i++)
                for (size_t j = 0; j < nk; j++) {
                    const float *qr = q + (q0 + i) * d, *kr = k + (kv0 + j) * kv_row_stride;
                    float acc = 0.0f;
                    for (size_t e = 0; e < d; e++) acc += qr[e] * kr[e];
                    s[i * BKV + j] = acc * scale;
                }
            if (mask) { /* :277-278 */
                for (size_t i = 0; i < nq; i++)
                    for (size_t j = 0; j < nk; j++)
                        s[i * BKV + j] += mask[(q0 + i) * mask_row_stride + kv0 + j];
            } else if (causal) { /* :279-288: triu(-inf, k) => -inf where j - i >= k */
                long kdiag = (long)q0 - (long)kv0 - (long)q_len + (long)kv_len + 1;
                for (size_t i = 0; i < nq; i++)
                    for (size_t j = 0; j < nk; j++)
                        s[i * BKV + j] += ((long)j - (long)i >= kdiag) ? -INFINITY : 0.0f;
            }
            for (size_t i = 0; i < nq; i++) {
                float *row = s + i * BKV;
                float tile_m = row[0]; /* :289-293 */
                for (size_t j = 1; j < nk; j++)
                    if (row[j] > tile_m) tile_m = row[j];
                if (isfinite(tile_m)) /* :294-298 */
                    for (size_t j = 0; j < nk; j++) row[j] -= tile_m;
                float tile_l = 0.0f;
                for (size_t j = 0; j < nk; j++) { /* :300-301 */
                    row[j] = expf(row[j]);
                    tile_l += row[j];
                }
                size_t qi = q0 + i;
                float m_new = fmaxf(m[qi], tile_m); /* :303, f32::max (NaN-ignoring, like fmaxf) */
                float e_old = expf(m[qi] - m_new), e_tile = expf(tile_m - m_new);
                float l_new = e_old * l[qi] + e_tile * tile_l; /* :305-310 */
                /* :314  sv = P . Vb */
                float *svr = sv + i * d;
                for (size_t e = 0; e < d; e++) svr[e] = 0.0f;
                for (size_t j = 0; j < nk; j++) {
                    const float *vr = v + (kv0 + j) * kv_row_stride;
                    float p = row[j];
                    for (size_t e = 0; e < d; e++) svr[e] += p * vr[e];
                }
                float r_l_new = 1.0f / l_new;            /* :316 */
                float mul_o = e_old * l[qi] * r_l_new;   /* :317 */
                float mul_sv = e_tile * r_l_new;         /* :318 */
                float *orow = out + qi * d;
                for (size_t e = 0; e < d; e++) orow[e] = orow[e] * mul_o + svr[e] * mul_sv; /* :321 */
                l[qi] = l_new; /* :330-331 */
                m[qi] = m_new;
            }
        }
    }
    free(l);
    free(m);
    free(s);
    free(sv);
}

/* FlashSdpaOp::flash_attention_gqa (flash_sdpa.rs:187-227): one task per
 * (batch, q_head), kv head = q_head / group (:200).  `threads` > 1 spreads the
 * tasks over an OpenMP team like rayon's global pool does (:209-221).
 * q [B,Hq,Sq,D] dense; k, v [B,Hkv,*,D] with strides (in floats) for batch, head
 * and token; mask optional [Mb,Mh,Sq,Sk] dense with broadcast dims of size 1
 * (batch/head index clamped like :251-252); scale < 0 selects 1/sqrt(D) (:246). */
ORC_API void orc_flash_sdpa_f32(const float *q, const float *k, const float *v, const float *mask,
                                size_t B, size_t Hq, size_t Hkv, size_t Sq, size_t Sk, size_t D,
                                size_t k_stride_b, size_t k_stride_h, size_t k_stride_t,
                                size_t mask_b, size_t mask_h, int causal, int has_scale,
                                float scale_in, float *out, int threads) {
    size_t group = Hq / Hkv;
    float scale = has_scale ? scale_in : sqrtf(1.0f / (float)D); /* :246 (d as f32).recip().sqrt() */
    long n_tasks = (long)(B * Hq);
    if (Sk == 0) {
        memset(out, 0, B * Hq * Sq * D * sizeof(float));
        return;
    }
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : 1)
#endif
    for (long t = 0; t < n_tasks; t++) {
        size_t b = (size_t)t / Hq, qh = (size_t)t % Hq, kvh = qh / group;
        const float *mk = NULL;
        if (mask) {
            size_t mb = b < mask_b - 1 ? b : mask_b - 1, mh = qh < mask_h - 1 ? qh : mask_h - 1;
            mk = mask + (mb * mask_h + mh) * Sq * Sk;
        }
        attend_one_head(q + (b * Hq + qh) * Sq * D, k + b * k_stride_b + kvh * k_stride_h,
                        v + b * k_stride_b + kvh * k_stride_h, k_stride_t, mk, Sk, Sq, Sk, D, causal,
                        scale, out + (b * Hq + qh) * Sq * D);
    }
    (void)threads;
}

/* FlashSdpaOp::eval (flash_sdpa.rs:103-163) for f16 tensors: cast the WHOLE of Q,
 * K and V to f32 (:111), attend, cast the result back to f16 (:162).  K/V are
 * dense [B,Hkv,Sk,D] here (that is what the op receives from the concat cache). */
ORC_API void orc_flash_sdpa_eval_f16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                     const uint16_t *mask, size_t B, size_t Hq, size_t Hkv,
                                     size_t Sq, size_t Sk, size_t D, size_t mask_b, size_t mask_h,
                                     int causal, int has_scale, float scale, uint16_t *out,
                                     int threads) {
    size_t nq = B * Hq * Sq * D, nk = B * Hkv * Sk * D;
    float *qf = (float *)malloc(nq * 4), *kf = (float *)malloc(nk * 4 + 4),
          *vf = (float *)malloc(nk * 4 + 4), *of = (float *)malloc(nq * 4), *mf = NULL;
    orc_f16_to_f32_n(q, qf, nq);
    orc_f16_to_f32_n(k, kf, nk);
    orc_f16_to_f32_n(v, vf, nk);
    if (mask) {
        size_t nm = mask_b * mask_h * Sq * Sk;
        mf = (float *)malloc(nm * 4);
        orc_f16_to_f32_n(mask, mf, nm);
    }
    orc_flash_sdpa_f32(qf, kf, vf, mf, B, Hq, Hkv, Sq, Sk, D, Hkv * Sk * D, Sk * D, D, mask_b, mask_h,
                       causal, has_scale, scale, of, threads);
    orc_f32_to_f16_n(of, out, nq);
    free(qf);
    free(kf);
    free(vf);
    free(of);
    free(mf);
}

/* Textbook softmax(Q K^T * scale + mask) V in f64 — the mathematical ground
 * truth used to pin the flash restatement (the reference's own closed-form test
 * reference is test-rt/suite-unit/src/sdpa.rs:187-236: causal masks c > p + r with
 * p = Sk - Sq, mask added after the causal fill).  Inputs are f32, output f64. */
ORC_API void orc_naive_sdpa_f64(const float *q, const float *k, const float *v, const float *mask,
                                size_t B, size_t Hq, size_t Hkv, size_t Sq, size_t Sk, size_t D,
                                size_t mask_b, size_t mask_h, int causal, int has_scale,
                                float scale_in, double *out) {
    size_t group = Hq / Hkv;
    double scale = has_scale ? (double)scale_in : 1.0 / sqrt((double)D);
    double *s = (double *)malloc((Sk ? Sk : 1) * sizeof(double));
    long p = (long)Sk - (long)Sq;
    if (p < 0) p = 0; /* saturating_sub, sdpa.rs(test):219 */
    for (size_t b = 0; b < B; b++)
        for (size_t qh = 0; qh < Hq; qh++) {
            size_t kvh = qh / group;
            const float *kk = k + (b * Hkv + kvh) * Sk * D, *vv = v + (b * Hkv + kvh) * Sk * D;
            const float *mk = NULL;
            if (mask) {
                size_t mb = b < mask_b - 1 ? b : mask_b - 1, mh = qh < mask_h - 1 ? qh : mask_h - 1;
                mk = mask + (mb * mask_h + mh) * Sq * Sk;
            }
            for (size_t i = 0; i < Sq; i++) {
                const float *qr = q + ((b * Hq + qh) * Sq + i) * D;
                double mx = -INFINITY;
                for (size_t j = 0; j < Sk; j++) {
                    double acc = 0.0;
                    for (size_t e = 0; e < D; e++) acc += (double)qr[e] * (double)kk[j * D + e];
                    acc *= scale;
                    if (causal && (long)j > p + (long)i) acc = -INFINITY;
                    if (mk) acc += (double)mk[i * Sk + j];
                    s[j] = acc;
                    if (acc > mx) mx = acc;
                }
                double sum = 0.0;
                for (size_t j = 0; j < Sk; j++) {
                    s[j] = exp(s[j] - mx);
                    sum += s[j];
                }
                double *o = out + ((b * Hq + qh) * Sq + i) * D;
                for (size_t e = 0; e < D; e++) {
                    double acc = 0.0;
                    for (size_t j = 0; j < Sk; j++) acc += s[j] * (double)vv[j * D + e];
                    o[e] = acc / sum;
                }
            }
        }
    free(s);
}

ORC_API int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* One decode step of the reference's default CPU path, costs included, for the
 * benchmark's cpu_baseline: DynKeyValueCache (concat: fresh allocation + copy of
 * the whole past, dyn_kv_cache.rs:158-174) for K and V, then FlashSdpaOp::eval on
 * f16 tensors (whole-tensor casts to f32, flash_sdpa.rs:103-163).
 * k_past/v_past: dense [B,Hkv,T,D] f16; k_new/v_new: [B,Hkv,1,D]; q: [B,Hq,1,D].
 * Returns newly allocated K and V ([B,Hkv,T+1,D], caller frees with orc_free). */
ORC_API void orc_decode_step_f16(const uint16_t *q, const uint16_t *k_past, const uint16_t *v_past,
                                 const uint16_t *k_new, const uint16_t *v_new, size_t B, size_t Hq,
                                 size_t Hkv, size_t T, size_t D, int threads, uint16_t *out,
                                 uint16_t **k_out, uint16_t **v_out) {
    uint16_t *kc = (uint16_t *)orc_concat_append((const uint8_t *)k_past, T, (const uint8_t *)k_new, 1,
                                                 B * Hkv, D * 2);
    uint16_t *vc = (uint16_t *)orc_concat_append((const uint8_t *)v_past, T, (const uint8_t *)v_new, 1,
                                                 B * Hkv, D * 2);
    orc_flash_sdpa_eval_f16(q, kc, vc, NULL, B, Hq, Hkv, 1, T + 1, D, 1, 1, 1, 0, 0.0f, out, threads);
    *k_out = kc;
    *v_out = vc;
}

/* ------------------------------------------------------------------------- */
/* RotateHalf and ApplyRope (transformers/src/ops/apply_rope.rs).              */
/* Dense row-major input of shape[0..rank), rank <= 4; cos/sin given with      */
/* element strides for the input's rank, 0 on broadcast axes.                  */
/* ------------------------------------------------------------------------- */

/* f16 * f16 and f16 + f16 as crate `half` computes them without native fp16
 * arithmetic: widen, operate in f32, round to f16. */
static inline uint16_t h_mul(uint16_t a, uint16_t b) { return orc_f32_to_f16(orc_f16_to_f32(a) * orc_f16_to_f32(b)); }
static inline uint16_t h_add(uint16_t a, uint16_t b) { return orc_f32_to_f16(orc_f16_to_f32(a) + orc_f16_to_f32(b)); }

/* apply_rope.rs:58-76: tensor[.., 0..h] = -input[.., h..]; tensor[.., h..] = input[.., 0..h] */
ORC_API void orc_rotate_half(int is_f16, const void *in, void *out, size_t rows, size_t inner) {
    size_t h = inner / 2;
    for (size_t r = 0; r < rows; r++) {
        if (is_f16) {
            const uint16_t *x = (const uint16_t *)in + r * inner;
            uint16_t *y = (uint16_t *)out + r * inner;
            for (size_t i = 0; i < h; i++) {
                y[i] = (uint16_t)(x[i + h] ^ 0x8000u); /* Neg flips the sign bit */
                y[i + h] = x[i];
            }
        } else {
            const float *x = (const float *)in + r * inner;
            float *y = (float *)out + r * inner;
            for (size_t i = 0; i < h; i++) {
                y[i] = -x[i + h];
                y[i + h] = x[i];
            }
        }
    }
}

/* apply_rope.rs:169-176: Add(Mul(input, cos), Mul(RotateHalf(input), sin)), each op in the
 * input's datum type with numpy-style broadcasting of cos and sin. */
ORC_API void orc_apply_rope(int is_f16, const void *in, const void *cosv, const void *sinv, void *out, int rank,
                            const size_t *shape, const size_t *cs_strides) {
    size_t sh[4] = {1, 1, 1, 1}, cs[4] = {0, 0, 0, 0};
    for (int d = 0; d < rank; d++) {
        sh[4 - rank + d] = shape[d];
        cs[4 - rank + d] = cs_strides[d];
    }
    size_t inner = sh[3], h = inner / 2;
    size_t rows = sh[0] * sh[1] * sh[2];
    void *rot = malloc(rows * inner * (is_f16 ? 2 : 4));
    orc_rotate_half(is_f16, in, rot, rows, inner);
    (void)h;
    for (size_t i0 = 0; i0 < sh[0]; i0++)
        for (size_t i1 = 0; i1 < sh[1]; i1++)
            for (size_t i2 = 0; i2 < sh[2]; i2++)
                for (size_t i3 = 0; i3 < sh[3]; i3++) {
                    size_t e = ((i0 * sh[1] + i1) * sh[2] + i2) * sh[3] + i3;
                    size_t c = i0 * cs[0] + i1 * cs[1] + i2 * cs[2] + i3 * cs[3];
                    if (is_f16) {
                        const uint16_t *x = in, *r = rot, *co = cosv, *si = sinv;
                        ((uint16_t *)out)[e] = h_add(h_mul(x[e], co[c]), h_mul(r[e], si[c]));
                    } else {
                        const float *x = in, *r = rot, *co = cosv, *si = sinv;
                        float a = x[e] * co[c];
                        float b = r[e] * si[c];
                        ((float *)out)[e] = a + b;
                    }
                }
    free(rot);
}

/* ------------------------------------------------------------------------- */
/* WindowKvCache (transformers/src/ops/window_kv_cache.rs:80-154): ring buffer  */
/* of `window` rows per (batch, head); rows are opaque byte strings.            */
/* ------------------------------------------------------------------------- */
typedef struct {
    size_t outer, window, row_bytes, len, cursor;
    unsigned char *buf; /* [outer][window][row_bytes], allocated on first push */
} orc_win;

ORC_API orc_win *orc_win_new(size_t outer, size_t window, size_t row_bytes) {
    orc_win *c = (orc_win *)calloc(1, sizeof(orc_win));
    c->outer = outer, c->window = window, c->row_bytes = row_bytes;
    return c;
}
ORC_API void orc_win_free(orc_win *c) {
    if (c) free(c->buf);
    free(c);
}
ORC_API size_t orc_win_len(const orc_win *c) { return c->len; }
ORC_API size_t orc_win_cursor(const orc_win *c) { return c->cursor; }
ORC_API size_t orc_win_capacity(const orc_win *c) { return c->buf ? c->window : 0; } /* :98-100 */

/* buf[.., dst0 .. dst0+n) = src[.., src0 .. src0+n) along the token axis (assign_slice) */
static void win_assign(orc_win *c, size_t dst0, const unsigned char *src, size_t n_new, size_t src0, size_t n) {
    for (size_t o = 0; o < c->outer; o++)
        memcpy(c->buf + (o * c->window + dst0) * c->row_bytes, src + (o * n_new + src0) * c->row_bytes, n * c->row_bytes);
}

/* push, :111-143.  src is [outer][n_new][row_bytes]. */
ORC_API void orc_win_push(orc_win *c, const void *srcv, size_t n_new) {
    const unsigned char *src = (const unsigned char *)srcv;
    if (n_new == 0) return;                                                       /* :113-115 */
    if (!c->buf) c->buf = (unsigned char *)malloc(c->outer * c->window * c->row_bytes); /* :101-108 */
    size_t w = c->window;
    if (n_new >= w) {                                                             /* :119-126 */
        win_assign(c, 0, src, n_new, n_new - w, w);
        c->cursor = 0;
        c->len = w;
        return;
    }
    size_t end = c->cursor + n_new;                                               /* :129 */
    if (end <= w) {
        win_assign(c, c->cursor, src, n_new, 0, n_new);
        c->cursor = end == w ? 0 : end;
    } else {
        size_t first = w - c->cursor;
        win_assign(c, c->cursor, src, n_new, 0, first);
        win_assign(c, 0, src, n_new, first, n_new - first);
        c->cursor = n_new - first;
    }
    c->len = c->len + n_new < w ? c->len + n_new : w;                             /* :141 */
}

/* valid_view, :145-152: slots [0, len) in physical order, copied out dense [outer][len][row_bytes] */
ORC_API void orc_win_valid(const orc_win *c, void *dstv) {
    unsigned char *dst = (unsigned char *)dstv;
    for (size_t o = 0; o < c->outer; o++)
        memcpy(dst + o * c->len * c->row_bytes, c->buf + o * c->window * c->row_bytes, c->len * c->row_bytes);
}

/* ------------------------------------------------------------------------- */
/* StreamedSdpaOp                                                               */
/* ------------------------------------------------------------------------- */

/* StreamedSdpaOp::flash_attention_gqa (transformers/src/ops/streamed_sdpa.rs:164-272): one query row at a
 * time over key blocks of `block_k`, f32 throughout (eval casts f16 inputs to f32 and the result back,
 * :112-160).  mask: optional [q_len, kv_len] shared by every batch and head (:143-152); with a mask the
 * causal flag is not consulted (:216-222); causal hides key i_k > t_q, counted from the first key whatever
 * kv_len is (:218).  A block whose largest score is not finite is skipped whole (:231-234), a score that is
 * not finite contributes nothing (:247-249), a row that saw nothing is zero (:263). */
ORC_API int orc_streamed_sdpa_f32(const float *q, const float *k, const float *v, const float *mask, size_t B, size_t Hq,
                          size_t Hkv, size_t Sq, size_t Sk, size_t D, int causal, int has_scale, float scale_in,
                          size_t block_k, float *out) {
    if (Hkv == 0 || Hq % Hkv) return 1;
    const float scale = has_scale ? scale_in : sqrtf(1.0f / (float)D); /* :183: recip().sqrt() */
    if (block_k < 1) block_k = 1;                                       /* :184 */
    const size_t group = Hq / Hkv;
    float *acc = (float *)malloc(D * sizeof(float));
    float *scores = (float *)malloc(block_k * sizeof(float));
    for (size_t b = 0; b < B; b++)
        for (size_t kh = 0; kh < Hkv; kh++) {
            const float *kbh = k + (b * Hkv + kh) * Sk * D, *vbh = v + (b * Hkv + kh) * Sk * D;
            for (size_t g = 0; g < group; g++) {
                const size_t qh = kh * group + g; /* :195 */
                for (size_t tq = 0; tq < Sq; tq++) {
                    const float *qv = q + ((b * Hq + qh) * Sq + tq) * D;
                    float m = -INFINITY, l = 0.0f; /* :203-205 */
                    for (size_t e = 0; e < D; e++) acc[e] = 0.0f;
                    for (size_t kb = 0; kb < Sk; kb += block_k) {
                        const size_t kend = kb + block_k < Sk ? kb + block_k : Sk;
                        float block_max = -INFINITY;
                        for (size_t ik = kb; ik < kend; ik++) {
                            const float mk = mask ? mask[tq * Sk + ik] : (causal && ik > tq) ? -INFINITY : 0.0f;
                            float dot = 0.0f; /* dot1d :275-282: serial f32 sum */
                            for (size_t e = 0; e < D; e++) dot += qv[e] * kbh[ik * D + e];
                            const float s = dot * scale + mk; /* :223 */
                            if (s > block_max) block_max = s;
                            scores[ik - kb] = s;
                        }
                        if (!isfinite(block_max)) continue; /* :231-234 */
                        const float new_m = m > block_max ? m : block_max;
                        const float alpha = isfinite(m) ? expf(m - new_m) : 0.0f; /* :237 */
                        if (alpha != 1.0f) {
                            for (size_t e = 0; e < D; e++) acc[e] *= alpha;
                            l *= alpha;
                        }
                        float block_l = 0.0f;
                        for (size_t ik = kb; ik < kend; ik++) {
                            const float s = scores[ik - kb];
                            if (!isfinite(s)) continue; /* :247-249 */
                            const float w = expf(s - new_m);
                            block_l += w;
                            for (size_t e = 0; e < D; e++) acc[e] += w * vbh[ik * D + e];
                        }
                        l += block_l;
                        m = new_m;
                    }
                    const float inv_l = l > 0.0f ? 1.0f / l : 0.0f; /* :263 */
                    float *o = out + ((b * Hq + qh) * Sq + tq) * D;
                    for (size_t e = 0; e < D; e++) o[e] = acc[e] * inv_l;
                }
            }
        }
    free(acc);
    free(scores);
    return 0;
}
