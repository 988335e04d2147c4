// MFMA prefill attention for gfx950, throughput version for q_len >= 32 (GQA heads share K/V tiles).
// f16 in/out, f32 accumulate, causal (bottom-right aligned), unmasked or with an additive mask input, GQA,
// K/V read in place.
//
// Same transposed formulation as sdpa_prefill.hip (S^T = K.Q^T, O^T = V^T.P^T with 32x32x16 MFMAs,
// every softmax scalar of a query in one lane).  What differs is how a compute unit is kept busy:
//
//  * One workgroup = 8 waves = 8 different (query head, 32-query block) pairs that all read the
//    SAME 64-key K/V tile: HG query heads of one kv head (GQA) x 8/HG query blocks.  A tile
//    staged into LDS once feeds 8 waves, so staging traffic per MFMA is a quarter of what a
//    one-head 64-query workgroup needs.
//  * K and V tiles are double buffered in LDS and fetched two tiles ahead through registers, so a
//    tile costs one barrier and the global-memory latency stays hidden.  (Running the two waves
//    of a SIMD half an iteration apart, so that one's softmax would overlap the other's MFMAs,
//    was tried and measured no faster: the hardware already interleaves them.)
//  * Few workgroups (small batch) are spread over the chip by splitting the key range over
//    several workgroups.  Each writes its normalised partial output in f16 plus (m, l) to the
//    workspace, laid out exactly as the accumulator registers are (so every store instruction
//    covers 512 contiguous bytes), and a small kernel merges them.
//  * The output accumulators are rescaled only when some query's running maximum moved.
//  * A second tile loop (template argument PING, chosen with TROCM_PREFILL_PING=1, f16 caches without a mask
//    input) loads K/V tiles straight into LDS (global_load_lds_dwordx4, swizzled rows) and runs waves 0..3 and
//    4..7 half a tile apart, one group on the matrix cores while the other computes its softmax.  It gives the
//    same results and, measured, the same speed (within 2 %) as the loop that stages through registers, which
//    stays the default: removing the barriers, the load waits or the priorities from it changes nothing, while
//    removing the MFMAs, the LDS fragment reads, the softmax or the direct loads shortens it by 36, 26, 18
//    and 12 %: the parts add up, because an MFMA in flight blocks most of the other wave's vector issue slots.
//
// Roofline: MFMA-bound.  FLOPs = 4 * B * Hq * D * (visible query-key pairs).
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include <type_traits>
#include <utility>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));

struct PrefillPP {
    const _Float16 *q;
    _Float16 *out;
    const _Float16 *k, *v;
    int64_t kv_stride_b, kv_stride_h, kv_stride_t;  // elements
    int B, Hq, Hkv, Sq, Sk;
    int causal;
    int n_qtiles, nsplit;
    float scale_log2;
    // Partials of key split s and 32-query block wb (= (b * Hq + qh) * n_qb32 + q / 32):
    _Float16 *part_o;   // [nsplit][n_wb][D / 4][32 queries][4 features], normalised by l
    float *part_ml;     // [nsplit][n_wb][2][32 queries]: m (log2 domain), then l
    int n_qb32;
    int64_t n_wb;
    // additive mask [mask_b, mask_h, Sq, Sk] of f16 (masked kernels only); element strides, 0 on a broadcast axis
    const _Float16 *mask;
    int64_t mask_stride_b, mask_stride_h;
    int mask_vec;       // rows allow 8-byte loads (Sk % 4 == 0 and an 8-byte aligned base)
    // != NULL: arrival counters, one per (batch, query tile, head group, kv head), zero between launches;
    // the last key split of a tile to arrive merges the partials itself and no merge launch follows
    int *counters;
    // Q8_0 / Q4_0 caches (kernels with FMT != TROCM_F16): code planes [B, Hkv, pitch, D or D/2] bytes at
    // k / v, f16 scale planes [B, Hkv, pitch, D/32]; strides in token rows
    const uint16_t *k_scales, *v_scales;
    int64_t row_stride_b, row_stride_h;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Transposing 64-bit LDS load of 16-bit elements: in each block of 16 lanes, lane i receives
// element i%4 of the four 8-byte rows addressed by lanes i/4, i/4+4, i/4+8, i/4+12.
__device__ __forceinline__ half4_t lds_read_tr16(const _Float16 *lds_ptr) {
    typedef __attribute__((address_space(3))) short4_t *lds_v4_ptr;
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(uintptr_t)(uint32_t)(uintptr_t)lds_ptr);
    return __builtin_bit_cast(half4_t, r);
}

constexpr int kWavesPP = 8, kThreadsPP = 64 * kWavesPP, kTileN = 64;

template <class F, int... Is>
__device__ __attribute__((always_inline)) inline void static_for_impl(F &&f, std::integer_sequence<int, Is...>) { (f(std::integral_constant<int, Is>{}), ...); }
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <int N, class F>
__device__ __attribute__((always_inline)) inline void static_for(F &&f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }
constexpr float kLazyMax = 8.0f;
#ifndef TROCM_PING_PRIO_MFMA
#define TROCM_PING_PRIO_MFMA 1
#endif
#ifndef TROCM_PING_DEPTH
#define TROCM_PING_DEPTH 4   // fragments requested ahead of the MFMA that uses them
#endif
#ifndef TROCM_PING_PRIO_VALU
#define TROCM_PING_PRIO_VALU 0
#endif

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// bytes (b0, b1) / (b2, b3) of a word as the half pairs (1024 + b): the byte under exponent byte 0x64
__device__ __forceinline__ half2_t magic_lo(uint32_t w) { return __builtin_bit_cast(half2_t, perm(0x64646464u, w, 0x04010400u)); }
__device__ __forceinline__ half2_t magic_hi(uint32_t w) { return __builtin_bit_cast(half2_t, perm(0x64646464u, w, 0x04030402u)); }

// Eight code bytes -> the reference's f16 dequantised values (code - zero) * d, each rounded once to
// f16 (q4_0.rs:82-95): (1024 + u) - (1024 + zero) is exact, the product rounds.
__device__ __forceinline__ u32x4 dequant8(uint32_t b0123, uint32_t b4567, half2_t zero1024, half2_t d2) {
    u32x4 r;
    r.x = __builtin_bit_cast(uint32_t, (magic_lo(b0123) - zero1024) * d2);
    r.y = __builtin_bit_cast(uint32_t, (magic_hi(b0123) - zero1024) * d2);
    r.z = __builtin_bit_cast(uint32_t, (magic_lo(b4567) - zero1024) * d2);
    r.w = __builtin_bit_cast(uint32_t, (magic_hi(b4567) - zero1024) * d2);
    return r;
}


template <int D, int HG, bool MASK, int FMT, bool PING = false>
__global__ __launch_bounds__(kThreadsPP) void sdpa_prefill_pp_kernel(PrefillPP p) {
    static_assert(!PING || (!MASK && FMT == TROCM_F16), "the ping-pong loop serves f16 caches without a mask input");
    constexpr int QB = kWavesPP / HG;     // 32-query blocks per workgroup
    constexpr int BLOCK_M = 32 * QB;
    constexpr int KS = D / 16;            // contraction steps of Q K^T
    constexpr int DB = D / 32;            // 32-feature blocks of the output
    constexpr int KROW = D + 8;           // halfs per K row in LDS: 128-bit reads of 16 rows hit 64 distinct banks
    constexpr int VROW = D + 16;          // halfs per V row in LDS: the 4 rows of a transposing read sit 8 banks apart
    constexpr int NL = kTileN * D / 8 / kThreadsPP;  // 128-bit loads per thread per tile and tensor
    static_assert(NL >= 1 && NL * 8 * kThreadsPP == kTileN * D, "tile loads must divide evenly");

    // One LDS block: two K tiles, then two V tiles.  The ping-pong loop keeps rows unpadded (the direct loads write
    // 1024 contiguous bytes per instruction) and swizzles their 16-byte pieces instead.
    constexpr int K_TILE = PING ? kTileN * D : kTileN * KROW;   // halves
    constexpr int V_TILE = PING ? kTileN * D : kTileN * VROW;
    constexpr int TR_HALVES = kWavesPP * 32 * (D / 2 + 8);      // output transposition area of the epilogue
    constexpr int WTS_HALVES = kWavesPP * 16 * 32 * 2;          // merge weights of the epilogue (floats)
    constexpr int LDS_HALVES = PING ? (2 * K_TILE + 2 * V_TILE > WTS_HALVES + TR_HALVES ? 2 * K_TILE + 2 * V_TILE : WTS_HALVES + TR_HALVES)
                                    : 2 * K_TILE + 2 * V_TILE;
    __shared__ __attribute__((aligned(1024))) _Float16 lds_all[LDS_HALVES];
    _Float16 (*lds_k)[K_TILE] = reinterpret_cast<_Float16 (*)[K_TILE]>(&lds_all[0]);
    _Float16 (*lds_v)[V_TILE] = reinterpret_cast<_Float16 (*)[V_TILE]>(&lds_all[2 * K_TILE]);

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hb = lane >> 5, l32 = lane & 31;

    // workgroup -> (kv head fastest: consecutive workgroup ids go round-robin to the 8 XCDs, so
    // one kv head's K/V stays in one XCD's L2), head group, key split, query tile (longest first)
    int id = blockIdx.x;
    const int kvh = id % p.Hkv;
    id /= p.Hkv;
    const int G = p.Hq / p.Hkv;
    const int gg = id % (G / HG);
    id /= (G / HG);
    const int split = id % p.nsplit;
    id /= p.nsplit;
    const int qt = p.n_qtiles - 1 - (id % p.n_qtiles);
    const int b = id / p.n_qtiles;
    const int qh = kvh * G + gg * HG + (w % HG);

    const int off = p.Sk - p.Sq;          // query i sees keys j <= i + off when causal
    const int q0 = qt * BLOCK_M + 32 * (w / HG);  // first query of this wave
    const int my_q = q0 + l32;
    const bool wave_has_queries = q0 < p.Sq;
    const _Float16 *qrow = p.q + (((int64_t)b * p.Hq + qh) * p.Sq + min(my_q, p.Sq - 1)) * D;
    const _Float16 *kbase = p.k + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    const _Float16 *vbase = p.v + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;

    // key tiles of this workgroup: its share of the tiles its last query sees
    const int wg_q_last = min(qt * BLOCK_M + BLOCK_M, p.Sq) - 1;
    const int last_key = p.causal ? min(p.Sk - 1, wg_q_last + off) : p.Sk - 1;
    const int n_kt = last_key / kTileN + 1;
    const int per = (n_kt + p.nsplit - 1) / p.nsplit;
    const int t_begin = split * per;
    const int n_it = max(0, min(n_kt, t_begin + per) - t_begin);
    const int wave_q_last = min(q0 + 31, p.Sq - 1);

    float m_run = -INFINITY, l_run = 0.0f;   // m_run in the log2 domain, already scaled
    float16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;

    half8_t qf[KS];
    u32x4 kpre[NL], vpre[NL];
    // Quantised caches: a thread fetches one unit of 16 elements of a key row per tile and tensor -- 16
    // code bytes (Q8_0) or the 8 bytes that hold elements j..j+7 and 16+j..16+j+7 of a block (Q4_0) --
    // plus the block's scale, and dequantises while staging.
    constexpr bool QUANT = FMT != TROCM_F16;
    constexpr int UPR = D / 16;                        // units per key row
    const bool q_active = tid < kTileN * UPR;          // D = 64: half the threads
    const int q_key = tid / UPR, q_unit = tid % UPR;
    uint16_t ksc = 0, vsc = 0;
    const uint8_t *kq = nullptr, *vq = nullptr;
    const uint16_t *ksp = nullptr, *vsp = nullptr;
    if constexpr (QUANT) {
        const int64_t plane_row = (int64_t)b * p.row_stride_b + (int64_t)kvh * p.row_stride_h;
        constexpr int RB = FMT == TROCM_Q8_0 ? D : D / 2;   // code bytes per token row
        kq = reinterpret_cast<const uint8_t *>(p.k) + plane_row * RB;
        vq = reinterpret_cast<const uint8_t *>(p.v) + plane_row * RB;
        ksp = p.k_scales + plane_row * (D / 32);
        vsp = p.v_scales + plane_row * (D / 32);
    }
    auto prefetch = [&](int kt) {
        if constexpr (!QUANT) {
#pragma unroll
            for (int j = 0; j < NL; j++) {
                int c = j * kThreadsPP + tid;
                int key = c / (D / 8), dc = c % (D / 8);
                int64_t row = min(kt * kTileN + key, p.Sk - 1);
                kpre[j] = *reinterpret_cast<const u32x4 *>(kbase + row * p.kv_stride_t + dc * 8);
                vpre[j] = *reinterpret_cast<const u32x4 *>(vbase + row * p.kv_stride_t + dc * 8);
            }
        } else if (q_active) {
            const int64_t row = min(kt * kTileN + q_key, p.Sk - 1);
            if constexpr (FMT == TROCM_Q8_0) {
                kpre[0] = *reinterpret_cast<const u32x4 *>(kq + row * D + q_unit * 16);
                vpre[0] = *reinterpret_cast<const u32x4 *>(vq + row * D + q_unit * 16);
            } else {   // unit u of a row: block u / 2, bytes 8 * (u % 2) .. + 8 of its 16 code bytes
                const uint2 kk = *reinterpret_cast<const uint2 *>(kq + row * (D / 2) + q_unit * 8);
                const uint2 vv = *reinterpret_cast<const uint2 *>(vq + row * (D / 2) + q_unit * 8);
                kpre[0].x = kk.x, kpre[0].y = kk.y, vpre[0].x = vv.x, vpre[0].y = vv.y;
            }
            ksc = ksp[row * (D / 32) + q_unit / 2];
            vsc = vsp[row * (D / 32) + q_unit / 2];
        }
    };
    auto stage = [&](int kbuf, int vbuf) {
        if constexpr (!QUANT) {
#pragma unroll
            for (int j = 0; j < NL; j++) {
                int c = j * kThreadsPP + tid;
                int key = c / (D / 8), dc = c % (D / 8);
                *reinterpret_cast<u32x4 *>(&lds_k[kbuf][key * KROW + dc * 8]) = kpre[j];
                *reinterpret_cast<u32x4 *>(&lds_v[vbuf][key * VROW + dc * 8]) = vpre[j];
            }
        } else if (q_active) {
            const half2_t kd = {__builtin_bit_cast(_Float16, ksc), __builtin_bit_cast(_Float16, ksc)};
            const half2_t vd = {__builtin_bit_cast(_Float16, vsc), __builtin_bit_cast(_Float16, vsc)};
            u32x4 ka, kb2, va, vb2;     // two chunks of 8 halves per tensor
            int dc_a, dc_b;             // their 16-byte chunk indices in the row
            if constexpr (FMT == TROCM_Q8_0) {
                const half2_t zero = {(_Float16)1152.0f, (_Float16)1152.0f};   // 1024 + 128: the plane holds code + 128
                ka = dequant8(kpre[0].x, kpre[0].y, zero, kd), kb2 = dequant8(kpre[0].z, kpre[0].w, zero, kd);
                va = dequant8(vpre[0].x, vpre[0].y, zero, vd), vb2 = dequant8(vpre[0].z, vpre[0].w, zero, vd);
                dc_a = 2 * q_unit, dc_b = 2 * q_unit + 1;
            } else {
                const half2_t zero = {(_Float16)1032.0f, (_Float16)1032.0f};   // 1024 + 8
                // low nibbles: elements j..j+7 of the block, high nibbles: elements 16+j..16+j+7
                const uint32_t m = 0x0F0F0F0Fu;
                ka = dequant8(kpre[0].x & m, kpre[0].y & m, zero, kd), kb2 = dequant8((kpre[0].x >> 4) & m, (kpre[0].y >> 4) & m, zero, kd);
                va = dequant8(vpre[0].x & m, vpre[0].y & m, zero, vd), vb2 = dequant8((vpre[0].x >> 4) & m, (vpre[0].y >> 4) & m, zero, vd);
                dc_a = 4 * (q_unit / 2) + (q_unit % 2), dc_b = dc_a + 2;
            }
            *reinterpret_cast<u32x4 *>(&lds_k[kbuf][q_key * KROW + dc_a * 8]) = ka;
            *reinterpret_cast<u32x4 *>(&lds_k[kbuf][q_key * KROW + dc_b * 8]) = kb2;
            *reinterpret_cast<u32x4 *>(&lds_v[vbuf][q_key * VROW + dc_a * 8]) = va;
            *reinterpret_cast<u32x4 *>(&lds_v[vbuf][q_key * VROW + dc_b * 8]) = vb2;
        }
    };

    // Mask values of this lane's query for the 32 keys it owns in a tile: 8 groups of 4 consecutive
    // keys, fetched one tile ahead (issued right after the previous tile's softmax has consumed them).
    half4_t mpre[MASK ? 8 : 1];
    const _Float16 *mrow = nullptr;
    if constexpr (MASK)
        mrow = p.mask + (int64_t)b * p.mask_stride_b + (int64_t)qh * p.mask_stride_h + (int64_t)min(my_q, p.Sq - 1) * p.Sk;
    auto prefetch_mask = [&](int kt) {
        if constexpr (MASK) {
#pragma unroll
            for (int g = 0; g < 8; g++) {
                const int key0 = kt * kTileN + 32 * (g >> 2) + 8 * (g & 3) + 4 * hb;
                if (p.mask_vec) {
                    mpre[g] = *reinterpret_cast<const half4_t *>(mrow + min(key0, p.Sk - 4));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) mpre[g][i] = mrow[min(key0 + i, p.Sk - 1)];
                }
            }
        }
    };

    // does this wave have anything to do on tile kt?
    auto tile_active = [&](int kt) __attribute__((always_inline)) { return wave_has_queries && (!p.causal || kt * kTileN <= wave_q_last + off); };

    // ---- S^T = K Q^T : 2 key blocks of 32 x 32 queries ---------------------------------------------
    auto qk = [&](int kbuf, float16_t (&s)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) s[kb][r] = 0.0f;
        const _Float16 *kt_base = &lds_k[kbuf][l32 * KROW + 8 * hb];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                half8_t kf = *reinterpret_cast<const half8_t *>(kt_base + (32 * kb) * KROW + 16 * ks);
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s[kb], 0, 0, 0);
            }
        }
    };

    // ---- online softmax for query lane%32 over this lane's 32 keys; leaves P^T fragments in pf ----
    auto softmax = [&](int kt, float16_t (&s)[2], half8_t (&pf)[4]) __attribute__((always_inline)) {
        const int k_lo = kt * kTileN;
        if constexpr (MASK) {
            // logits in the log2 domain, mask added: the maximum below is then taken after the scaling
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    s[kb][r] = __builtin_fmaf((float)mpre[4 * kb + (r >> 2)][r & 3], 1.4426950408889634f, s[kb][r] * p.scale_log2);
        }
        const bool need_mask = (k_lo + kTileN > p.Sk) || (p.causal && (k_lo + kTileN - 1 > q0 + off));
        if (need_mask) {
            // key k_lo + 4 hb + c, c = 32 kb + 8 (r / 4) + r % 4, is visible when c <= lim
            const int lim = (p.causal ? min(p.Sk - 1, my_q + off) : p.Sk - 1) - k_lo - 4 * hb;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) s[kb][r] = (32 * kb + 8 * (r >> 2) + (r & 3)) <= lim ? s[kb][r] : -INFINITY;
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) tmax = fmaxf(tmax, s[kb][r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        // The reference of the exponentials follows the maximum lazily: it moves only when this tile's maximum exceeds it
        // by more than kLazyMax (the exponentials then reach 2^kLazyMax at most, far inside f16 and f32 range), so the
        // accumulators are rescaled a few times per sequence instead of at most tiles; o / l does not depend on it.
        const float t_scaled = MASK ? tmax : tmax * p.scale_log2;   // scale > 0: the maximum commutes with the scaling
        const bool moved = t_scaled > m_run + kLazyMax;   // also the first visible key (reference -inf); never for a maximum of -inf
        const float m_new = moved ? t_scaled : m_run;
        const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // nothing visible yet: keep everything at zero
        float psum = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float sx = s[st >> 1][8 * (st & 1) + i];
                float pv = fast_exp2(MASK ? sx - m_ref : __builtin_fmaf(sx, p.scale_log2, -m_ref));
                pf[st][i] = (_Float16)pv;
            }
            // the row sum is taken over the f16 values that enter the product with V (one v_dot2 per pair
            // instead of two additions, and numerator and denominator see the same rounding)
            const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t pair = {pf[st][2 * i], pf[st][2 * i + 1]};
                psum = __builtin_amdgcn_fdot2(pair, ones, psum, false);
            }
        }
        const float alpha = moved ? fast_exp2(m_run - m_ref) : 1.0f;   // 0 from a reference of -inf
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        }
    };

    // ---- O^T += V^T P^T ---------------------------------------------------------------------------------
    // This lane as a SOURCE of the transposing loads: key row (lane%16)/4 of a group of four,
    // features 16*(lane/16 % 2) + 4*(lane%4) of the 32-feature block.
    const int vsrc_off = (4 * hb + ((lane & 15) >> 2)) * VROW + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    auto pv = [&](int vbuf, half8_t (&pf)[4]) {
        const _Float16 *vsrc = &lds_v[vbuf][vsrc_off];
#pragma unroll
        for (int st = 0; st < 4; st++) {
#pragma unroll
            for (int db = 0; db < DB; db++) {
                half4_t lo = lds_read_tr16(vsrc + (16 * st) * VROW + 32 * db);      // keys 16st + 4hb + 0..3
                half4_t hi = lds_read_tr16(vsrc + (16 * st + 8) * VROW + 32 * db);  // keys 16st + 8 + 4hb + 0..3
                half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[st], o[db], 0, 0, 0);
            }
        }
    };

    if constexpr (!PING) {
        if (n_it > 0) prefetch(t_begin);   // issued before the Q loads: both latencies overlap
        // Q^T fragments: query = lane % 32, features 16*ks + 8*hb .. +8
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qf[ks] = *reinterpret_cast<const half8_t *>(qrow + 16 * ks + 8 * hb);
        // Settle the Q loads here.  Otherwise the compiler must assume they may still be in flight at
        // the top of the tile loop and waits for vmcnt(0) at their first use there, which also waits
        // for the K/V prefetch issued a few instructions earlier and exposes its whole latency.
#pragma unroll
        for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[ks]));

        if (n_it > 0) {
            stage(0, 0);
            if (n_it > 1) prefetch(t_begin + 1);
            prefetch_mask(t_begin);
        }
        for (int it = 0; it < n_it; it++) {
            __syncthreads();   // tile `it` is in LDS; every wave is done with the buffers about to be overwritten
            const int cur = it & 1;
            const int kt = t_begin + it;
            if (tile_active(kt)) {
                float16_t s[2];
                half8_t pf[4];
                qk(cur, s);
                softmax(kt, s, pf);
                if (it + 1 < n_it) prefetch_mask(kt + 1);
                pv(cur, pf);
            }
            // The next tile goes to LDS after this one's arithmetic, not before it: its loads were issued a whole
            // iteration ago in the steady state and right before the loop for the first iteration, whose arithmetic
            // then covers their latency.
            if (it + 1 < n_it) {
                stage(cur ^ 1, cur ^ 1);
                if (it + 2 < n_it) prefetch(t_begin + it + 2);
            }
        }
    } else {
        // ---- ping-pong loop -----------------------------------------------------------------------------
        // Waves 0..3 and waves 4..7 (one of each per SIMD) run half a tile apart: while one group issues the 32 MFMAs
        // of P.V (previous tile) and K.Q^T (this tile), the other computes its softmax on the vector ALUs, and the
        // two swap at a barrier (two barriers per tile).  K and V tiles go from global memory straight into LDS
        // (global_load_lds_dwordx4: each lane fetches 16 bytes from its own address, the 64 pieces of an
        // instruction land in 1024 consecutive bytes), so rows are unpadded and bank conflicts are avoided by
        // storing the 16-byte piece p of row r at piece p ^ f(r): the lane that fills physical piece pp of row r
        // fetches logical piece pp ^ f(r).  f_k(r) = r % 16 (a K fragment read takes one piece of 16
        // consecutive rows per quarter wave), f_v(r) = 4 (r % 4) (a transposing V read takes 64 consecutive
        // bytes of 4 consecutive rows per half wave); with 128-byte rows (head size 64) r / 2 takes r's place.
        constexpr int ROWB = 2 * D, PPR = D / 8, RSH = D == 128 ? 0 : 1;
        constexpr int NLD = kTileN * PPR / 64 / kWavesPP;   // direct loads per wave, tile and tensor
        static_assert(NLD >= 1 && NLD * 64 * kWavesPP == kTileN * PPR, "tile pieces must divide over the waves");
        typedef __attribute__((address_space(3))) void *lds_void_ptr;
        typedef __attribute__((address_space(1))) const void *global_void_ptr;
        const int grp = w >> 2;
        const uint32_t lds0 = (uint32_t)(uintptr_t)&lds_all[0];
        // This lane's pieces of a tile: instruction n of wave w fills LDS bytes [(w NLD + n) 1024, + 1024) of the
        // tile, lane i the 16 bytes at 16 i: row (w NLD + n) (64 / PPR) + i / PPR, physical piece i % PPR.
        const int64_t row_bytes = p.kv_stride_t * 2;
        uint32_t koff[NLD], voff[NLD];   // byte offsets from the tile's first row (the host admits rows of less than 2^25 bytes)
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            const int row = (w * NLD + n) * (64 / PPR) + lane / PPR, pp = lane % PPR;
            koff[n] = (uint32_t)row * (uint32_t)row_bytes + (pp ^ ((row >> RSH) & (PPR - 1))) * 16;
            voff[n] = (uint32_t)row * (uint32_t)row_bytes + (pp ^ (4 * ((row >> RSH) & (PPR / 4 - 1)))) * 16;
        }
        // rows past the last key repeat the last key's row (their scores are masked; V must stay finite)
        auto clamped_off = [&](int kt, int n, bool is_v) __attribute__((always_inline)) {
            const int row = (w * NLD + n) * (64 / PPR) + lane / PPR, pp = lane % PPR;
            const int f = is_v ? 4 * ((row >> RSH) & (PPR / 4 - 1)) : (row >> RSH) & (PPR - 1);
            return (uint32_t)min(row, p.Sk - 1 - kt * kTileN) * (uint32_t)row_bytes + (uint32_t)((pp ^ f) * 16);
        };
        // keeps the 32-bit offset a 32-bit register up to the load (hoisted out of the loop it becomes a 64-bit one)
        auto opaque = [](uint32_t v) __attribute__((always_inline)) {
            asm volatile("" : "+v"(v));
            return v;
        };
        auto issue_k = [&](int kt, int buf) __attribute__((always_inline)) {
            const char *tile = reinterpret_cast<const char *>(kbase) + (int64_t)kt * kTileN * row_bytes;
            const bool whole = (kt + 1) * kTileN <= p.Sk;
#pragma unroll
            for (int n = 0; n < NLD; n++)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(tile + opaque(whole ? koff[n] : clamped_off(kt, n, false))),
                                                 (lds_void_ptr)(uintptr_t)(lds0 + (uint32_t)((buf * K_TILE) * 2 + (w * NLD + n) * 1024)), 16, 0, 0);
        };
        auto issue_v = [&](int kt, int buf) __attribute__((always_inline)) {
            const char *tile = reinterpret_cast<const char *>(vbase) + (int64_t)kt * kTileN * row_bytes;
            const bool whole = (kt + 1) * kTileN <= p.Sk;
#pragma unroll
            for (int n = 0; n < NLD; n++)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(tile + opaque(whole ? voff[n] : clamped_off(kt, n, true))),
                                                 (lds_void_ptr)(uintptr_t)(lds0 + (uint32_t)((2 * K_TILE + buf * V_TILE) * 2 + (w * NLD + n) * 1024)), 16, 0, 0);
        };
        // tile it + 1's K and tile it's V: both buffers were last read two barriers ago
        auto issue_loads = [&](int it) __attribute__((always_inline)) {
            if (it + 1 < n_it) issue_k(t_begin + it + 1, (it + 1) & 1);
            if (it < n_it) issue_v(t_begin + it, it & 1);
        };
        auto loads_landed = []() __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        };

        // K fragment of (key block kb, step ks): row 32 kb + lane % 32, logical piece 2 ks + hb
        const uint32_t kfrag = lds0 + l32 * ROWB + ((hb ^ ((l32 >> RSH) & (PPR - 1))) << 4);
        // Per-lane LDS byte addresses of the K fragments of step ks (key block 0) and of the V^T fragments of
        // feature block db (keys 0..7) in the buffers the next matrix half reads; they flip after every iteration.
        uint32_t kx[KS], vx[DB];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kx[ks] = kfrag ^ (uint32_t)(ks << 5);
        // V^T fragments: this lane as a source of the transposing loads addresses key row 4 hb + (lane % 16) / 4 of
        // a group of 8, features 16 (lane / 16 % 2) + 4 (lane % 4) of the 32-feature block db
        const int vrl = 4 * hb + ((lane & 15) >> 2);
        const uint32_t vfrag = lds0 + (2 * K_TILE + V_TILE) * 2 + vrl * ROWB +
                               (((2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) ^ (4 * ((vrl >> RSH) & (PPR / 4 - 1)))) << 4) + 8 * (lane & 1);
#pragma unroll
        for (int db = 0; db < DB; db++) vx[db] = vfrag ^ (uint32_t)(db << 6);   // iteration 1 reads tile 0 in buffer 0 after one flip
        int kflip = K_TILE * 2, vflip = -V_TILE * 2;   // bytes to the other buffer
        auto flip_buffers = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kx[ks] += (uint32_t)kflip;
#pragma unroll
            for (int db = 0; db < DB; db++) vx[db] += (uint32_t)vflip;
            kflip = -kflip, vflip = -vflip;
        };

        float16_t s[2];
        half8_t pf[4];
        // The matrix half of an iteration: the 4 DB fragments of V^T and the MFMAs of P.V (when DO_PV), then the 2 KS
        // fragments of K and the MFMAs of K.Q^T (when DO_QK).  The LDS reads are written out (with their waits)
        // because the compiler, which cannot tell the direct loads' LDS writes from the tiles being read, would
        // wait for every direct load before the first read, and because it keeps only one or two reads in flight:
        // here fragment i + kDepth is requested before fragment i is used.  LDS reads return in order, so the wait
        // before fragment i's MFMA allows as many outstanding reads as were issued after its own.
        auto matrix_half = [&](auto pv_tag, auto qk_tag) __attribute__((always_inline)) {
            constexpr bool DO_PV = decltype(pv_tag)::value, DO_QK = decltype(qk_tag)::value;
            constexpr int NV = DO_PV ? 4 * DB : 0, NK = DO_QK ? 2 * KS : 0, NF = NV + NK;
            constexpr int PD = TROCM_PING_DEPTH < NF ? TROCM_PING_DEPTH : NF;
            half4_t vlo[DO_PV ? 4 * DB : 1], vhi[DO_PV ? 4 * DB : 1];
            half8_t kf[DO_QK ? 2 * KS : 1];
            auto request = [&](auto ic) __attribute__((always_inline)) {
                (void)vlo, (void)vhi, (void)kf, (void)vx, (void)kx;   // named outside the dependent branches, so that they are captured
                constexpr int i = decltype(ic)::value;
                if constexpr (i < NV) {
                    constexpr int off = 16 * (i / DB) * ROWB;
                    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vlo[i]) : "v"(vx[i % DB]), "n"(off));
                    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vhi[i]) : "v"(vx[i % DB]), "n"(off + 8 * ROWB));
                } else {
                    constexpr int j = i - NV;
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[j]) : "v"(kx[j / 2]), "n"((j % 2) * 32 * ROWB));
                }
            };
            static_for<PD>(request);
            static_for<NF>([&](auto ic) __attribute__((always_inline)) {
                (void)vlo, (void)vhi, (void)kf, (void)s, (void)pf, (void)qf, (void)o;
                constexpr int i = decltype(ic)::value;
                if constexpr (i + PD < NF) request(std::integral_constant<int, i + PD>{});
                constexpr int last = i + PD < NF ? i + PD : NF - 1;      // the last fragment requested so far
                constexpr int behind = (last < NV ? 2 * (last - i) : i < NV ? 2 * (NV - 1 - i) + (last - NV + 1) : last - i);
                if constexpr (i < NV) {
                    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(vlo[i]), "+v"(vhi[i]) : "n"(behind));
                    const half8_t vf = __builtin_shufflevector(vlo[i], vhi[i], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[i % DB] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[i / DB], o[i % DB], 0, 0, 0);
                } else {
                    constexpr int j = i - NV;
                    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(kf[j]) : "n"(behind));
                    if constexpr (j < 2) {
#pragma unroll
                        for (int r = 0; r < 16; r++) s[j % 2][r] = 0.0f;
                    }
                    s[j % 2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[j], qf[j / 2], s[j % 2], 0, 0, 0);
                }
            });
        };
        // barrier without a fence: a fence would wait for the direct loads in flight (they count as LDS writes)
        auto half_barrier = []() __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        };

        if (n_it > 0) issue_k(t_begin, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qf[ks] = *reinterpret_cast<const half8_t *>(qrow + 16 * ks + 8 * hb);
        loads_landed();
#pragma unroll
        for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[ks]));
        half_barrier();   // the first K tile is in LDS
        if (grp == 1) {    // the second group starts half a tile late
            issue_loads(0);
            half_barrier();
        }
        // Iteration `it`, matrix half: P.V of tile it - 1, then K.Q^T of tile it; vector half: softmax of tile it.
        // Every wave issues its share of the loads of (K of tile it + 1, V of tile it) at the start of the first
        // group's matrix half and waits for them before the barrier that ends the second group's: they have two
        // half-tiles to land.  Every wave takes every tile of the workgroup: a tile that a wave's queries do not see
        // (or a wave without queries) comes out of the softmax as all zeros.  The first and the last iteration,
        // which lack one of the two products, are written out on their own, so that no two versions of the
        // accumulators meet after a branch.
        auto iteration = [&](int it, auto pv_tag, auto qk_tag) __attribute__((always_inline)) {
            if (grp == 0) issue_loads(it);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(TROCM_PING_PRIO_MFMA);
            matrix_half(pv_tag, qk_tag);
            __builtin_amdgcn_s_setprio(TROCM_PING_PRIO_VALU);
            if (grp == 1) loads_landed();
            half_barrier();
            if (grp == 1) issue_loads(it + 1);
            if constexpr (decltype(qk_tag)::value) softmax(t_begin + it, s, pf);
            flip_buffers();
            if (grp == 0) loads_landed();
            half_barrier();
        };
        if (n_it > 0) {
            iteration(0, std::false_type{}, std::true_type{});
            for (int it = 1; it < n_it; it++) iteration(it, std::true_type{}, std::true_type{});
            iteration(n_it, std::true_type{}, std::false_type{});
        }
        if (grp == 0) half_barrier();   // as many barriers as the second group
    }
    l_run += __shfl_xor(l_run, 32, 64);
    // Output rows of this wave (32 queries of one head: one contiguous block of 32 * D halves).  A lane holds
    // 4-feature pieces of its own query's row, which stored as they stand would touch 32 rows per instruction;
    // they go through a wave-private corner of the (idle) V tile buffers instead, half of the features at a
    // time, and leave as 16-byte pieces of consecutive addresses.  Callers make sure every wave of the
    // workgroup is past the tile loop.
    auto wave_sync = []() {   // orders this wave's LDS accesses across its lanes (no instruction: the LDS serves a wave in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    auto write_output = [&](float mul) {
        constexpr int FP = D / 2, TROW = FP + 8, CPRW = FP / 8, RPI = 64 / CPRW;   // features per pass, LDS row, 16-byte pieces per row, rows per instruction
        static_assert(kWavesPP * 32 * TROW == TR_HALVES && (PING || TR_HALVES <= 2 * V_TILE), "transposition area exceeds the V tile buffers");
        _Float16 *tr = (PING ? &lds_all[WTS_HALVES] : &lds_v[0][0]) + w * (32 * TROW);
        _Float16 *obase = p.out + (((int64_t)b * p.Hq + qh) * p.Sq + q0) * D;
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int d2 = 0; d2 < DB / 2; d2++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    half4_t h4;
#pragma unroll
                    for (int i = 0; i < 4; i++) h4[i] = (_Float16)(o[h * (DB / 2) + d2][4 * rq + i] * mul);
                    *reinterpret_cast<half4_t *>(tr + l32 * TROW + 32 * d2 + 8 * rq + 4 * hb) = h4;
                }
            wave_sync();   // lanes read what other lanes of the wave wrote
#pragma unroll
            for (int i = 0; i < 32 / RPI; i++) {
                const int row = i * RPI + lane / CPRW, ch = lane % CPRW;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(tr + row * TROW + ch * 8);
                if (q0 + row < p.Sq) *reinterpret_cast<u32x4 *>(obase + (int64_t)row * D + h * FP + ch * 8) = v;
            }
            wave_sync();   // ... and are done reading before the second half overwrites it
        }
    };
    if (p.nsplit == 1) {
        __syncthreads();   // the V tile buffers are idle from here on
        if (!wave_has_queries) return;
        write_output(l_run > 0.0f ? 1.0f / l_run : 0.0f);
        return;
    }
    // ---- key splits: store this split's normalised partial -----------------------------------------
    // With arrival counters the stores are agent-scope write-through stores: they are visible to every
    // compute unit of the device once they complete, so no cache write-back is needed before the
    // workgroup signals its arrival.
    const bool tail_merge = p.counters != nullptr;
    const int64_t wb = ((int64_t)b * p.Hq + qh) * p.n_qb32 + (q0 >> 5);
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    // An element of this split's normalised partial, as it is stored.  The product is rounded to f32 on its own
    // and then to f16, here and wherever the value is formed again (the merge below takes the own split's
    // values from the accumulators): the multiplication is written out so that the compiler cannot fuse the two
    // steps in one place and not in the other, which would round differently in rare cases (and, being volatile,
    // stays where it is used instead of being hoisted, all 64 products at once, above the merge's loads).
    auto partial_elem = [&](float acc) {
        float pr;
        asm volatile("v_mul_f32 %0, %1, %2" : "=v"(pr) : "v"(acc), "v"(inv));
        return (_Float16)pr;
    };
    if (wave_has_queries) {
        _Float16 *po = p.part_o + ((int64_t)split * p.n_wb + wb) * (32 * D) + l32 * 4;
        float *pml = p.part_ml + ((int64_t)split * p.n_wb + wb) * 64 + lane;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                half4_t h4;
#pragma unroll
                for (int i = 0; i < 4; i++) h4[i] = partial_elem(o[db][4 * rq + i]);
                _Float16 *dst = po + (8 * db + 2 * rq + hb) * 128;
                if (tail_merge)
                    __hip_atomic_store(reinterpret_cast<uint64_t *>(dst), __builtin_bit_cast(uint64_t, h4), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                else
                    *reinterpret_cast<half4_t *>(dst) = h4;
            }
        if (tail_merge)
            __hip_atomic_store(pml, hb ? l_run : m_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            *pml = hb ? l_run : m_run;
    }
    if (!tail_merge) return;

    // ---- the last split of this tile to arrive merges all of them ------------------------------------
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial stores have completed
    __syncthreads();                                     // ... and so have the whole workgroup's
    __shared__ int s_last;
    if (tid == 0) {
        int *counter = p.counters + (((int64_t)b * p.n_qtiles + qt) * (G / HG) + gg) * p.Hkv + kvh;
        const int arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = arrived == p.nsplit - 1;
        if (s_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    }
    __syncthreads();
    if (!s_last || !wave_has_queries) return;
    // Every wave merges its own 32-query block: out = sum_s w_s O_s, w_s = l_s 2^(m_s - max m) / sum.
    // The weights go through a wave-private corner of the (now idle) K tile buffer; the partial
    // outputs are laid out as the accumulators are, so each lane reads back exactly its own elements,
    // two splits in flight at a time.
    constexpr int kMaxSplits = 16;
    auto aload_f = [](const float *a) { return __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    static_assert(kWavesPP * kMaxSplits * 32 * sizeof(float) == WTS_HALVES * sizeof(_Float16) && WTS_HALVES <= 2 * K_TILE, "merge weights exceed the K tile buffers");
    float *wts = reinterpret_cast<float *>(&lds_all[0]) + w * (kMaxSplits * 32);
    // One merge step for NS splits starting at s0: their outputs and, when WEIGHTS, the (m, l) records of
    // MAXS splits are requested together; the weights go through LDS (lanes 32..63 need those of lanes 0..31).
    auto load_outputs = [&](int s0, auto &raw, auto ns_tag) {
        constexpr int NS = decltype(ns_tag)::value;
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const _Float16 *po = p.part_o + ((int64_t)min(s0 + j, p.nsplit - 1) * p.n_wb + wb) * (32 * D) + l32 * 4;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++)
                    raw[j][db * 4 + rq] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(po + (8 * db + 2 * rq + hb) * 128),
                                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    // Every lane works out the weights of its query into lv (lanes l and l + 32 the same ones, from the same
    // loads): nothing is handed from lane to lane.
    auto weights = [&](auto maxs_tag, auto &lv) {
        constexpr int MAXS = decltype(maxs_tag)::value;
        float mv[MAXS];
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            const float *ml = p.part_ml + ((int64_t)min(sp, p.nsplit - 1) * p.n_wb + wb) * 64;
            mv[sp] = aload_f(ml + l32);
            lv[sp] = aload_f(ml + 32 + l32);
        }
        float mm = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) mm = fmaxf(mm, mv[sp]);
        const float m_ref = (mm == -INFINITY) ? 0.0f : mm;
        float total = 0.0f;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            lv[sp] = sp < p.nsplit ? lv[sp] * fast_exp2(mv[sp] - m_ref) : 0.0f;
            total += lv[sp];
        }
        const float inv_total = total > 0.0f ? 1.0f / total : 0.0f;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) lv[sp] *= inv_total;
    };
    auto accumulate = [&](int s0, auto &raw, auto ns_tag) {
        constexpr int NS = decltype(ns_tag)::value;
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const float wgt = s0 + j < p.nsplit ? wts[(s0 + j) * 32 + l32] : 0.0f;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const half4_t h4 = __builtin_bit_cast(half4_t, raw[j][db * 4 + rq]);
#pragma unroll
                    for (int i = 0; i < 4; i++) o[db][4 * rq + i] += wgt * (float)h4[i];
                }
        }
    };
    auto zero_o = [&]() {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    };
    if (p.nsplit <= 4) {
        // The common case: everything in one round trip to the L2, and this workgroup's own partial, still in
        // its accumulators, is not read back.  Every element is the chain fma(w3, O3, fma(w2, O2, fma(w1, O1,
        // w0 O0))) over the splits in their order, the own term entering at its place with the f16 value that
        // was stored: the result does not depend on which split arrived last.
        uint64_t raw[3][DB * 4];   // the other splits in their order
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int sj = min(j + (j >= split), p.nsplit - 1);
            const _Float16 *po = p.part_o + ((int64_t)sj * p.n_wb + wb) * (32 * D) + l32 * 4;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++)
                    raw[j][db * 4 + rq] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(po + (8 * db + 2 * rq + hb) * 128),
                                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        float wv[4];   // 0 past the last split
        weights(std::integral_constant<int, 4>{}, wv);
        auto chain = [&](auto own_tag) {
            constexpr int K = decltype(own_tag)::value;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    half4_t h[3];
#pragma unroll
                    for (int j = 0; j < 3; j++) h[j] = __builtin_bit_cast(half4_t, raw[j][db * 4 + rq]);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float mine = (float)partial_elem(o[db][4 * rq + i]);
                        float acc = 0.0f;
#pragma unroll
                        for (int sp = 0; sp < 4; sp++) {
                            const float term = sp == K ? mine : (float)h[sp < K ? sp : sp - 1][i];
                            acc = sp == 0 ? wv[0] * term : __builtin_fmaf(wv[sp], term, acc);
                        }
                        o[db][4 * rq + i] = acc;
                    }
                    __builtin_amdgcn_sched_barrier(0);   // piece by piece: hoisting all the own-term products at once spills
                }
        };
        switch (split) {
            case 0: chain(std::integral_constant<int, 0>{}); break;
            case 1: chain(std::integral_constant<int, 1>{}); break;
            case 2: chain(std::integral_constant<int, 2>{}); break;
            default: chain(std::integral_constant<int, 3>{}); break;
        }
    } else {
        float wv[kMaxSplits];
        weights(std::integral_constant<int, kMaxSplits>{}, wv);
#pragma unroll
        for (int sp = 0; sp < kMaxSplits; sp++) wts[sp * 32 + l32] = wv[sp];   // lanes l and l + 32 write the same value and read it back
        zero_o();
        for (int s0 = 0; s0 < p.nsplit; s0 += 2) {
            uint64_t raw[2][DB * 4];
            load_outputs(s0, raw, std::integral_constant<int, 2>{});
            accumulate(s0, raw, std::integral_constant<int, 2>{});
        }
    }
    write_output(1.0f);
}

// Merge of the key splits, one workgroup per 32-query block:
//   out = sum_s w_s O_s / sum_s w_s,   w_s = l_s 2^(m_s - max m),   O_s normalised partial outputs.
template <int D>
__global__ __launch_bounds__(256) void sdpa_prefill_merge_kernel(PrefillPP p) {
    constexpr int kMaxSplits = 16;
    constexpr int OROW = D + 8;
    __shared__ float wts[kMaxSplits][32];
    __shared__ __attribute__((aligned(16))) _Float16 tile[32 * OROW];
    const int64_t wb = blockIdx.x;
    const int tid = threadIdx.x;
    if (tid < 32) {
        float mm = -INFINITY;
        for (int sp = 0; sp < p.nsplit; sp++) mm = fmaxf(mm, p.part_ml[((int64_t)sp * p.n_wb + wb) * 64 + tid]);
        const float m_ref = (mm == -INFINITY) ? 0.0f : mm;
        float total = 0.0f;
        for (int sp = 0; sp < p.nsplit; sp++) {
            const float *ml = p.part_ml + ((int64_t)sp * p.n_wb + wb) * 64;
            const float wgt = ml[32 + tid] * fast_exp2(ml[tid] - m_ref);
            wts[sp][tid] = wgt;
            total += wgt;
        }
        const float inv = total > 0.0f ? 1.0f / total : 0.0f;
        for (int sp = 0; sp < p.nsplit; sp++) wts[sp][tid] *= inv;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < D / 32; j++) {
        const int idx = j * 256 + tid;       // (feature group, query) in the partials' order
        const int fg = idx >> 5, q = idx & 31;
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int sp = 0; sp < p.nsplit; sp++) {
            const half4_t h = *reinterpret_cast<const half4_t *>(p.part_o + ((int64_t)sp * p.n_wb + wb) * (32 * D) + idx * 4);
            const float wgt = wts[sp][q];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] += wgt * (float)h[i];
        }
        half4_t h4;
#pragma unroll
        for (int i = 0; i < 4; i++) h4[i] = (_Float16)acc[i];
        *reinterpret_cast<half4_t *>(&tile[q * OROW + fg * 4]) = h4;
    }
    __syncthreads();
    const int64_t bh = wb / p.n_qb32;
    const int q_first = (int)(wb % p.n_qb32) * 32;
#pragma unroll
    for (int j = 0; j < D / 64; j++) {
        const int idx = j * 256 + tid;       // (query, 16-byte segment of its row)
        const int q = idx / (D / 8), seg = idx % (D / 8);
        if (q_first + q < p.Sq)
            *reinterpret_cast<u32x4 *>(p.out + (bh * p.Sq + q_first + q) * D + seg * 8) =
                *reinterpret_cast<const u32x4 *>(&tile[q * OROW + seg * 8]);
    }
}

int env_int(const char *name, int dflt) {
    const char *e = getenv(name);
    return e ? atoi(e) : dflt;
}

// TROCM_PREFILL_PING=0 keeps the loop that stages tiles through registers for f16 caches as well
bool ping_enabled() {
    static const int on = env_int("TROCM_PREFILL_PING", 0);
    return on != 0;
}

template <int D, int HG>
int launch_cfg(const PrefillPP &p, int fmt, int64_t wgs, hipStream_t s) {
    if (fmt == TROCM_Q8_0)
        hipLaunchKernelGGL((sdpa_prefill_pp_kernel<D, HG, false, TROCM_Q8_0>), dim3((unsigned)wgs), dim3(kThreadsPP), 0, s, p);
    else if (fmt == TROCM_Q4_0)
        hipLaunchKernelGGL((sdpa_prefill_pp_kernel<D, HG, false, TROCM_Q4_0>), dim3((unsigned)wgs), dim3(kThreadsPP), 0, s, p);
    else if (p.mask)
        hipLaunchKernelGGL((sdpa_prefill_pp_kernel<D, HG, true, TROCM_F16>), dim3((unsigned)wgs), dim3(kThreadsPP), 0, s, p);
    else if (ping_enabled())
        hipLaunchKernelGGL((sdpa_prefill_pp_kernel<D, HG, false, TROCM_F16, true>), dim3((unsigned)wgs), dim3(kThreadsPP), 0, s, p);
    else
        hipLaunchKernelGGL((sdpa_prefill_pp_kernel<D, HG, false, TROCM_F16>), dim3((unsigned)wgs), dim3(kThreadsPP), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_prefill_pp launch failed: %s", hipGetErrorString(e));
    if (p.nsplit > 1 && p.counters == nullptr) {
        hipLaunchKernelGGL((sdpa_prefill_merge_kernel<D>), dim3((unsigned)p.n_wb), dim3(256), 0, s, p);
        e = hipGetLastError();
        if (e != hipSuccess) return fail("sdpa_prefill_merge launch failed: %s", hipGetErrorString(e));
    }
    return 0;
}

template <int D>
int launch_hg(const PrefillPP &p, int fmt, int hg, int64_t wgs, hipStream_t s) {
    switch (hg) {
        case 4: return launch_cfg<D, 4>(p, fmt, wgs, s);
        case 2: return launch_cfg<D, 2>(p, fmt, wgs, s);
        default: return launch_cfg<D, 1>(p, fmt, wgs, s);
    }
}

}  // namespace

static size_t split_bytes(int64_t n_wb, int64_t D) { return (size_t)n_wb * (32 * (size_t)D * sizeof(_Float16) + 64 * sizeof(float)); }

// Upper bound of the partial-result area the staggered prefill kernel may use for this shape.
size_t prefill_workspace_bytes(int64_t B, int64_t Hq, int64_t Sq, int64_t D) {
    if (Sq < 2 || (D != 64 && D != 128)) return 0;
    const int64_t wgs1 = B * ((Hq + 3) / 4) * ((Sq + 63) / 64);  // about the fewest workgroups any head grouping gives
    const int64_t cus = 256;
    if (wgs1 >= cus) return 0;
    int64_t ns = (cus + wgs1 - 1) / wgs1;
    if (ns > 16) ns = 16;
    return (size_t)ns * split_bytes(B * Hq * ((Sq + 31) / 32), D) + 256;
}

int launch_sdpa_prefill_pp(const SdpaArgs &a, hipStream_t s) {
    if (a.q_dtype != TROCM_F16) return 2;
    const bool quant = is_quant(a.kv_fmt);
    if (!quant && a.kv_fmt != TROCM_F16) return 2;
    if (quant && (a.mask || a.kv_stride_t != a.D || !a.k_scales || !a.v_scales)) return 2;   // cache planes: dense token rows
    if (a.mask && a.causal) return 2;
    if (a.D != 128 && a.D != 64) return 2;
    if (a.Sq < 2 || a.Sk < 1 || a.Hq % a.Hkv) return 2;
    if (!(a.scale > 0.0f)) return 2;       // the running maximum is taken before scaling
    if (a.causal && a.Sk < a.Sq) return 2;  // some queries would see nothing: the generic kernel owns that case
    if (a.Sk >= (1ll << 30) || a.Sq >= (1ll << 30) || a.B >= (1ll << 20)) return 2;
    if ((a.kv_stride_b % 8) || (a.kv_stride_h % 8) || (a.kv_stride_t % 8)) return 2;  // 128-bit row loads
    if (a.kv_stride_t >= (1ll << 24)) return 2;  // byte offsets within a tile are 32-bit
    if ((uintptr_t)a.q % 16 || (uintptr_t)a.k % 16 || (uintptr_t)a.v % 16 || (uintptr_t)a.out % 16) return 2;
    if (quant) {   // strides arrive in elements of the logical [.., D] rows: whole token rows per head and batch
        if (a.kv_stride_h % a.D || a.kv_stride_b % a.D) return 2;
        const int64_t rb = a.kv_fmt == TROCM_Q8_0 ? a.D : a.D / 2;
        if (((a.kv_stride_h / a.D) * rb) % 16 || ((a.kv_stride_b / a.D) * rb) % 16) return 2;
        if ((uintptr_t)a.k_scales % 2 || (uintptr_t)a.v_scales % 2) return 2;
    }
    static const int enabled = env_int("TROCM_PREFILL_PP", 1);
    if (!enabled) return 2;
    static const int forced_hg = env_int("TROCM_PREFILL_HG", 0);
    static const int forced_split = env_int("TROCM_PREFILL_SPLITS", 0);
    const int64_t G = a.Hq / a.Hkv;
    int hg = G % 4 == 0 ? 4 : G % 2 == 0 ? 2 : 1;
    if (forced_hg && G % forced_hg == 0 && (forced_hg == 1 || forced_hg == 2 || forced_hg == 4)) hg = forced_hg;
    const int block_m = 32 * kWavesPP / hg;
    const int64_t n_qtiles = (a.Sq + block_m - 1) / block_m;
    // Waves whose 32-query block lies past q_len idle.  With several heads per workgroup that is still
    // the better kernel for a few queries over a long cache (speculative decoding, tiny chunks): the
    // K/V tiles are read once per kv head instead of once per query head (8 x 32 heads x 4 queries over
    // 8192 tokens: 66 us against 183 us).  With one head per workgroup short prompts go to the smaller kernel.
    // (Quantised caches have no smaller kernel: they stay here whatever the prompt length.)
    if (hg == 1 && !quant && a.Sq * 2 < n_qtiles * block_m) return 2;

    PrefillPP p;
    memset(&p, 0, sizeof(p));
    p.q = (const _Float16 *)a.q;
    p.out = (_Float16 *)a.out;
    p.k = (const _Float16 *)a.k;
    p.v = (const _Float16 *)a.v;
    p.kv_stride_b = a.kv_stride_b, p.kv_stride_h = a.kv_stride_h, p.kv_stride_t = a.kv_stride_t;
    if (quant) {
        p.k_scales = (const uint16_t *)a.k_scales, p.v_scales = (const uint16_t *)a.v_scales;
        p.row_stride_b = a.kv_stride_b / a.D, p.row_stride_h = a.kv_stride_h / a.D;
    }
    p.B = (int)a.B, p.Hq = (int)a.Hq, p.Hkv = (int)a.Hkv, p.Sq = (int)a.Sq, p.Sk = (int)a.Sk;
    p.causal = a.causal;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    p.n_qtiles = (int)n_qtiles;
    p.n_qb32 = (int)((a.Sq + 31) / 32);
    p.n_wb = a.B * a.Hq * p.n_qb32;
    if (a.mask) {   // [mask_b, mask_h, Sq, Sk] dense
        p.mask = (const _Float16 *)a.mask;
        p.mask_stride_h = a.mask_h > 1 ? a.Sq * a.Sk : 0;
        p.mask_stride_b = a.mask_b > 1 ? a.mask_h * a.Sq * a.Sk : 0;
        p.mask_vec = a.Sk % 4 == 0 && (uintptr_t)a.mask % 8 == 0;
    }

    const int64_t wgs1 = a.B * (a.Hq / hg) * n_qtiles;
    const int64_t cus = num_compute_units();
    int64_t ns = 1;
    if (wgs1 < cus) {
        ns = (cus + wgs1 - 1) / wgs1;
        const int64_t tiles = (a.Sk + kTileN - 1) / kTileN;
        if (ns > tiles / 2) ns = tiles / 2;   // at least two tiles per split
        if (ns > 16) ns = 16;
    }
    if (forced_split > 0) ns = forced_split < 16 ? forced_split : 16;   // the merges handle at most 16 splits
    const size_t per_split = split_bytes(p.n_wb, a.D);
    const size_t avail = a.workspace && a.workspace_bytes > kWsCounterBytes + 256 ? a.workspace_bytes - kWsCounterBytes - 256 : 0;
    if (ns > 1 && (size_t)ns * per_split > avail) ns = (int64_t)(avail / per_split);
    if (ns < 1) ns = 1;
    p.nsplit = (int)ns;
    if (ns > 1) {
        char *base = (char *)a.workspace + kWsCounterBytes;
        base += (256 - ((uintptr_t)base & 255)) & 255;
        p.part_o = (_Float16 *)base;
        p.part_ml = (float *)(base + (size_t)ns * p.n_wb * 32 * a.D * sizeof(_Float16));
        // With few enough tiles for the counter area the last split to arrive merges (no second launch);
        // TROCM_PREFILL_TAIL_MERGE=0 keeps the merge launch.
        static const int tail_merge = env_int("TROCM_PREFILL_TAIL_MERGE", 1);
        if (tail_merge && ns <= 16 && wgs1 <= (int64_t)(kWsCounterBytes / sizeof(int))) p.counters = (int *)a.workspace;
    }
    const int64_t wgs = wgs1 * ns;
    if (wgs >= (1ll << 31)) return 2;
    return a.D == 128 ? launch_hg<128>(p, a.kv_fmt, hg, wgs, s) : launch_hg<64>(p, a.kv_fmt, hg, wgs, s);
}

}  // namespace trocm
