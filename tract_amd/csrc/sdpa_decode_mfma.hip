// Split-K flash-decode attention with grouped query heads (q_len == 1, 2..32 query heads per kv head, f16
// queries) over f16, Q8_0 or Q4_0 caches, dense or ragged batches: gfx950.
//
// The vector-ALU decode kernel (sdpa_decode.hip) spends one v_dot2 per (head, 2 features) and one fma
// per (head, feature) of every token; with 8 heads per kv head that is about 970 vector instructions
// per wave and 32-token tile, and the kernel is bound by them, not by HBM (batch 8, 8192 tokens:
// 84.5 us against 47 us for 4 heads per kv head).  Here the G query heads of a kv head are the
// *columns* of MFMA tiles: S^T = K.Q^T and O^T = V^T.P^T, the same transposed formulation as the prefill
// kernel, with a head where that kernel has a query.  Only G of a tile's 16 (v_mfma_f32_16x16x32_f16, up
// to 16 heads) or 32 (v_mfma_f32_32x32x16_f16) columns are live, which the matrix pipe absorbs easily;
// what matters is that the vector work per tile drops to the softmax of 8 or 16 values per lane.
//
// Work decomposition: grid (splits, kv_heads, batch) or (work items, kv_heads), 4 waves; wave w takes
// 32-token tiles w, w+4, ... of its range.  Per tile: K rows global -> registers (one tile ahead,
// non-temporal) -> a wave-private LDS tile (block-quantised rows are dequantised on the way) -> A
// fragments; softmax in registers; V rows the same way into the same LDS tile (K is dead by then) ->
// transposing LDS reads -> A fragments of the second product.  Waves are merged through LDS, splits through
// the workspace: by the last workgroup to arrive (up to 8 heads per kv head, up to 32 splits) or by the merge
// launch, both shared with the other decode kernels.  A step's new token can be handed in and is stored to
// the cache by the kernel (f16 caches); an additive mask row per head can join the scores (f16 caches).
//
// Block-quantised caches at head_dim 128 with up to 16 heads per kv head do not dequantise at all: the raw codes go
// into the matrix cores as exact f16 integers, one 32-deep product per quantisation block, and the block scales are
// applied to the products (decode_mfma_qblock_body).
//
// Roofline: HBM-bound (f16) / bound by vector-instruction issue and the latency of a tile's dependent chain
// (quantised).  Algorithmic bytes as for sdpa_decode.hip and sdpa_decode_quant.hip.
#include <type_traits>
#include "decode_common.h"
#include "quant_block.h"

namespace trocm {
namespace {

typedef float float16_t __attribute__((ext_vector_type(16)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Transposing 64-bit LDS load of 16-bit elements: in each block of 16 lanes, lane i receives
// element i%4 of the four 8-byte rows addressed by lanes i/4, i/4+4, i/4+8, i/4+12.
__device__ __forceinline__ half4_t lds_read_tr16(const _Float16 *lds_ptr) {
    typedef __attribute__((address_space(3))) short4_t *lds_v4_ptr;
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(uintptr_t)(uint32_t)(uintptr_t)lds_ptr);
    return __builtin_bit_cast(half4_t, r);
}

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
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

// The power of two 2^-e that takes a positive finite x = m 2^e (m in [1/2, 1)) into [1/2, 1); 1 for zero, infinities and NaN.
__device__ __forceinline__ float pow2_normaliser(float x) {
    if (!(x > 0.0f) || x > 3.0e38f) return 1.0f;
    int e;
    (void)frexpf(x, &e);
    e = e > 126 ? 126 : (e < -126 ? -126 : e);   // the factor itself stays an ordinary float
    return ldexpf(1.0f, -e);
}

// What one workgroup has to do: a tile range of one (sequence, kv head), and where its result goes.
struct MfmaWork {
    int seq, kvh;                 // the sequence (batch entry) and kv head
    const char *kbase, *vbase;    // K and V rows of this (sequence, kv head): f16 rows or block codes
    const char *ksbase, *vsbase;  // quantised formats: their f16 block scales, D/32 per token
    int T, tile_begin, tile_end;
    int tile_step;                // a wave's next tile: kWaves (a contiguous range) or kWaves * splits (the splits of a
                                  // dense sequence-head take groups of kWaves tiles in turn)
    int skew_period, skew_split;  // > 0 (f16 body, interleaved splits, an even number of them): in every skew_period-th
                                  // round of groups the odd splits take none and their even neighbours two.  Workgroups go
                                  // to the 8 XCDs in turn, so odd splits run on odd XCDs, which stream about a tenth slower.
    int nsplit;                   // splits of this sequence-head (1: write the output rows)
    int64_t slot;                 // partial record of this workgroup
    int new_pos;                  // token stored by a fused append (-1: none)
    int *counter;                 // in-kernel merge by the last workgroup to arrive (dense batches, GP <= 8)
    int64_t part_first, part_stride;   // partial records of this sequence-head: first, first + stride, ...
    const char *mask;             // additive mask row of this kv head's first query head, token 0 (MASK instantiations)
};

// The tail every formulation shares: the four waves' records (O[GP][D], m[GP], l[GP], in `lds_raw`, kCombStride floats
// each) become the output rows (one split), or this workgroup's partial record, merged by the last workgroup to
// arrive or by the merge launch.
template <int D, int GP>
__device__ __forceinline__ void wave_records_to_output(const DecodeDev &p, const MfmaWork &wk, unsigned char *lds_raw, int64_t head0,
                                                       int g, int tid) {
    constexpr int kCombStride = GP * D + 2 * GP;
    float *comb = reinterpret_cast<float *>(lds_raw);   // [kWaves][GP*D + 2*GP]
    __syncthreads();
    __half *out = reinterpret_cast<__half *>(p.out) + head0 * D;
    const int64_t slot = wk.slot;
    // Rows of padded heads are neither combined nor stored when at most half the rows are real.  The merges of up to
    // kTailMergeMax splits then skip them too; the merge launch reads the rows of real heads only anyway; the wide merge
    // reads every row (its loads carry no condition) and writes the real ones: what it finds in rows 4..7 goes nowhere.
    const bool half_live = p.live_trim && GP == 8 && g <= GP / 2;
    const int rows_end = half_live ? (GP / 2) * D : GP * D;
    // two consecutive elements per thread: 64-bit LDS reads and 64-bit stores (the in-kernel merges of up to kTailMergeMax
    // splits read the records the same way)
    for (int idx = 2 * tid; idx < rows_end; idx += 2 * kThreads) {
        const int h = idx / D;
        float mm = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) mm = fmaxf(mm, comb[ww * kCombStride + GP * D + h]);
        const float mm_ref = mm == -INFINITY ? 0.0f : mm;   // a wave without tiles holds (0, -inf, 0)
        float acc0 = 0.0f, acc1 = 0.0f, ll = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
            const float f = fast_exp2(comb[ww * kCombStride + GP * D + h] - mm_ref);
            const float2 o2 = *reinterpret_cast<const float2 *>(comb + ww * kCombStride + idx);
            acc0 += o2.x * f, acc1 += o2.y * f;
            ll += comb[ww * kCombStride + GP * D + GP + h] * f;
        }
        if (wk.nsplit == 1) {
            if (h < g) {
                const float inv = ll > 0.0f ? 1.0f : 0.0f;
                out[idx] = __float2half_rn(inv != 0.0f ? acc0 / ll : 0.0f);
                out[idx + 1] = __float2half_rn(inv != 0.0f ? acc1 / ll : 0.0f);
            }
        } else if (wk.counter == nullptr) {
            *reinterpret_cast<float2 *>(p.part_o + slot * (GP * D) + idx) = float2{acc0, acc1};
            if ((idx % D) == 0) {
                p.part_ml[slot * (2 * GP) + h] = mm;
                p.part_ml[slot * (2 * GP) + GP + h] = ll;
            }
        } else {   // write-through stores: visible device-wide when they complete (see tail_merge)
            const uint64_t both = (uint64_t)__builtin_bit_cast(uint32_t, acc0) | ((uint64_t)__builtin_bit_cast(uint32_t, acc1) << 32);
            __hip_atomic_store(reinterpret_cast<uint64_t *>(p.part_o + slot * (GP * D) + idx), both, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((idx % D) == 0) {
                __hip_atomic_store(&p.part_ml[slot * (2 * GP) + h], mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&p.part_ml[slot * (2 * GP) + GP + h], ll, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if constexpr (GP <= 8) {   // (larger groups: the merge launch; the in-kernel merge would need too many registers)
        if (wk.nsplit > kTailMergeMax && wk.counter != nullptr)
            tail_merge_wide<__half, D, GP>(p, wk.counter, wk.nsplit, wk.part_first, wk.part_stride, out, tid, reinterpret_cast<float *>(lds_raw));
        else if (wk.nsplit > 1 && wk.nsplit <= 4 && wk.counter != nullptr && half_live)   // (cfg2's shape: 4 splits of 4 heads)
            tail_merge_pairs<__half, D, GP, GP / 2, 4>(p, wk.counter, wk.nsplit, wk.part_first, wk.part_stride, out, tid);
        else if (wk.nsplit > 1 && wk.counter != nullptr && half_live)
            tail_merge_pairs<__half, D, GP, GP / 2, kTailMergeMax>(p, wk.counter, wk.nsplit, wk.part_first, wk.part_stride, out, tid);
        else if (wk.nsplit > 1 && wk.counter != nullptr)
            tail_merge_pairs<__half, D, GP, GP, kTailMergeMax>(p, wk.counter, wk.nsplit, wk.part_first, wk.part_stride, out, tid);
    }
}

// FMT: TROCM_F16, or a block-quantised cache (TROCM_Q8_0 / TROCM_Q4_0, 32-element blocks): the codes are
// dequantised on the way into the LDS tile, (code - zero) * d rounded once to f16 as the reference's
// dequantisation rounds it, and everything after the tile is the f16 kernel.
// MASK: an additive mask [mask_b, mask_h, 1, T] of f16 joins the scaled scores (f16 caches, dense batches).
// W16: the tiles are 16 heads wide (v_mfma_f32_16x16x32_f16, up to 16 heads per kv head): half the matrix time,
// half the accumulator and query registers, and a lane exponentiates 8 scores instead of 16.  A lane then owns
// head lane % 16 and, of a 32-token tile, tokens 4*(lane/16) + 0..3 and 16 + 4*(lane/16) + 0..3; of the output,
// features 16*fb + 4*(lane/16) + 0..3 of every 16-feature block fb.
// Eight consecutive elements of a row rotated as ApplyRope does (apply_rope.rs:169-176): y = x * cos + RotateHalf(x) * sin,
// RotateHalf(x)[i] = -x[i + D/2] in the first half of the row and x[i - D/2] in the second, every product and the sum
// rounded to f16 (the products pass through an empty asm: this file is compiled with contraction on, and a fused
// multiply-add would round once where the CPU op rounds twice).  `row` / `cosr` / `sinr`: the D halves of the row and of
// its cos / sin rows; dc: which 16-byte chunk.
template <int D>
__device__ __forceinline__ u32x4 rope_chunk(const char *row, const char *cosr, const char *sinr, int dc) {
    constexpr int CPR = D / 8;
    const bool first = dc < CPR / 2;
    const half8_t x = *reinterpret_cast<const half8_t *>(row + dc * 16);
    const half8_t y = *reinterpret_cast<const half8_t *>(row + (first ? dc + CPR / 2 : dc - CPR / 2) * 16);
    const half8_t c = *reinterpret_cast<const half8_t *>(cosr + dc * 16), sn = *reinterpret_cast<const half8_t *>(sinr + dc * 16);
    half8_t a = x * c, b = (first ? -y : y) * sn;
    asm("" : "+v"(a), "+v"(b));   // (not volatile: several pieces' loads may be in flight together)
    return __builtin_bit_cast(u32x4, a + b);
}

// N consecutive elements (N = 4 or 8, not straddling the middle of the row) of a row of 128 halves, rotated the same way.
template <int N>
struct RopeRaw {
    typedef _Float16 vec_t __attribute__((ext_vector_type(N)));
    vec_t x, y, c, sn;   // the piece, its partner half a row away (sign applied), its cos and sin
};
template <int N>
__device__ __forceinline__ RopeRaw<N> rope_load128(const _Float16 *row, const char *cosr, const char *sinr, int f0) {
    typedef typename RopeRaw<N>::vec_t vec_t;
    const bool first = f0 < 64;
    RopeRaw<N> r;
    r.x = *reinterpret_cast<const vec_t *>(row + f0);
    const vec_t y = *reinterpret_cast<const vec_t *>(row + (first ? f0 + 64 : f0 - 64));
    r.y = first ? -y : y;
    r.c = *reinterpret_cast<const vec_t *>(cosr + 2 * f0), r.sn = *reinterpret_cast<const vec_t *>(sinr + 2 * f0);
    return r;
}
template <int N>
__device__ __forceinline__ typename RopeRaw<N>::vec_t rope_finish(const RopeRaw<N> &r) {
    typename RopeRaw<N>::vec_t a = r.x * r.c, b = r.y * r.sn;
    asm("" : "+v"(a), "+v"(b));   // (not volatile: volatile statements keep their order, and eight pieces would be eight round trips)
    return a + b;
}
template <int N>
__device__ __forceinline__ auto rope_piece128(const _Float16 *row, const char *cosr, const char *sinr, int f0) {
    return rope_finish<N>(rope_load128<N>(row, cosr, sinr, f0));
}

template <int D, int GP, int FMT, bool MASK = false, bool W16 = false, bool ROPE = false>
__device__ __forceinline__ void decode_mfma_body(const DecodeDev &p, const MfmaWork &wk) {
    static_assert(!W16 || GP <= 16, "the 16-wide layout: at most 16 heads");
    static_assert(!ROPE || (W16 && FMT == TROCM_F16 && !MASK), "the rotation is built for f16 rows on the 16-wide tiles");
    constexpr bool QUANT = FMT != TROCM_F16;
    constexpr int KS = D / 16;             // contraction steps of K.Q^T
    constexpr int DB = D / 32;             // 32-feature blocks of the output
    constexpr int KROW = D + 8;            // halfs per K row in LDS (128-bit reads of 16 rows hit distinct banks)
    constexpr int VROW = D + 16;           // halfs per V row in LDS (rows of a transposing read 8 banks apart)
    constexpr int RB = FMT == TROCM_F16 ? D * 2 : FMT == TROCM_Q8_0 ? D : D / 2;   // bytes per row in the cache
    constexpr int CPR = RB / 16;           // 16-byte chunks per row
    constexpr int EPC = D / CPR;           // elements per chunk: 8, 16 (Q8_0), 32 (Q4_0, one block)
    constexpr int NLD = kTile * CPR / 64;  // 128-bit loads per lane, tile and tensor
    constexpr int SROW = D / 32 * 2;       // bytes of block scales per row
    constexpr int kCombStride = GP * D + 2 * GP;
    constexpr int kTileBytes = kTile * VROW * 2;
    constexpr int kLdsBytes = kWaves * (kTileBytes > kCombStride * 4 ? kTileBytes : kCombStride * 4);
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLdsBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hb = lane >> 5;
    const int l16 = lane & 15, q4 = lane >> 4;
    const int hcol = W16 ? l16 : l32;   // the head (column of the score tile) of this lane
    const int kvh = wk.kvh, b = wk.seq;
    const int g = p.g_real;
    _Float16 *tile = reinterpret_cast<_Float16 *>(lds_raw + w * kTileBytes);

    const int64_t head0 = (int64_t)b * p.Hq + (int64_t)kvh * g;
    const _Float16 *qrow = reinterpret_cast<const _Float16 *>(p.q) + (head0 + min(hcol, g - 1)) * D;
    const char *kbase = wk.kbase, *vbase = wk.vbase;
    const int T = wk.T;
    const int tile_begin = wk.tile_begin, tile_end = wk.tile_end;

    // this lane's chunks of a tile: chunk j*64 + lane = (row, 16-byte chunk of the row)
    uint32_t g_off[NLD], k_slot[NLD], v_slot[NLD], s_off[QUANT ? NLD : 1];
#pragma unroll
    for (int j = 0; j < NLD; j++) {
        const int c = j * 64 + lane, row = c / CPR, dc = c % CPR;
        s_off[QUANT ? j : 0] = row * (D / 32 * 2);
        g_off[j] = (uint32_t)row * (uint32_t)p.kv_stride_t + (uint32_t)dc * 16u;
        k_slot[j] = row * KROW + dc * EPC;
        v_slot[j] = row * VROW + dc * EPC;
    }
    u32x4 kpre[NLD], vpre[NLD];
    // quantised: the 32-bit word that holds the scale of this lane's chunk (the chunk's place in its row, and
    // so the word and the half of it, is the same for every j), and the byte selector that doubles that half
    uint32_t ksc[QUANT ? NLD : 1], vsc[QUANT ? NLD : 1];
    const int my_block = (lane % CPR) * EPC / 32;
    const uint32_t sc_word = (my_block >> 1) * 4, sc_sel = (my_block & 1) ? 0x03020302u : 0x01000100u;
    // fused append: the row of token new_pos comes from the step's input wherever a tile holds it, and the first wave
    // of the sequence-head's first workgroup stores it to the cache here, ahead of the tile loop.  (Stored from inside
    // the loop, by the wave whose tile holds it, the store shared the vector-memory counter with the prefetches: the
    // compiler sizes a wait for the path with the fewest operations in flight, so every tile of every wave waited for
    // its newest loads as well -- 1.6 us of a 47.6 us launch, with or without a new token.)
    const int new_pos = wk.new_pos;
    const int64_t new_row = ((int64_t)b * p.Hkv + kvh) * D * 2;
    // (ROPE: the step's q and k_new rows are rotated on the way in, with the sequence's cos / sin rows)
    const char *cos_row = ROPE ? p.rope_cos + (int64_t)b * p.rope_stride_b : nullptr;
    const char *sin_row = ROPE ? p.rope_sin + (int64_t)b * p.rope_stride_b : nullptr;
    if constexpr (!QUANT) {
        if (new_pos >= 0 && w == 0 && wk.tile_begin == 0 && lane < 2 * CPR) {
            const int dc = lane % CPR;
            const char *src = (lane < CPR ? p.k_new : p.v_new) + new_row + dc * 16;
            char *dst = const_cast<char *>(lane < CPR ? kbase : vbase) + (int64_t)new_pos * p.kv_stride_t + dc * 16;
            u32x4 val = *reinterpret_cast<const u32x4 *>(src);
            if constexpr (ROPE) {
                if (lane < CPR) val = rope_chunk<D>(p.k_new + new_row, cos_row, sin_row, dc);
            }
            *reinterpret_cast<u32x4 *>(dst) = val;
        }
    }
    auto fetch_q = [&](const char *base0, const char *sbase0, int t, u32x4 (&dst)[NLD], uint32_t (&sc)[QUANT ? NLD : 1]) {
        const int t0 = t * kTile;
        const char *base = base0 + (int64_t)t0 * RB;
        const char *sbase = sbase0 + (int64_t)t0 * SROW + sc_word;
        if (t0 + kTile <= T) {   // whole tile: a wave-uniform base and this lane's fixed offsets
#pragma unroll
            for (int j = 0; j < (QUANT ? NLD : 0); j++) {
                dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + g_off[j]));
                sc[j] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sbase + s_off[QUANT ? j : 0]));
            }
        } else {
            const int last = T - 1 - t0;   // rows past the end of the sequence repeat its last token (masked below)
#pragma unroll
            for (int j = 0; j < (QUANT ? NLD : 0); j++) {
                const int c = j * 64 + lane, row = min(c / CPR, last), dc = c % CPR;
                dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + row * RB + dc * 16));
                sc[j] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sbase + row * SROW));
            }
        }
    };
    // codes of one tile -> f16 rows in the LDS tile
    auto stash_q = [&](const u32x4 (&codes)[NLD], const uint32_t (&sc)[QUANT ? NLD : 1], const uint32_t (&slot)[NLD]) {
#pragma unroll
        for (int j = 0; j < (QUANT ? NLD : 0); j++) {
            const half2_t d2 = __builtin_bit_cast(half2_t, perm(sc[j], sc[j], sc_sel));
            const u32x4 c = codes[j];
            if constexpr (FMT == TROCM_Q8_0) {
                const half2_t zero = {(_Float16)1152.0f, (_Float16)1152.0f};   // 1024 + 128: the plane holds code + 128
                *reinterpret_cast<u32x4 *>(tile + slot[j]) = dequant8(c.x, c.y, zero, d2);
                *reinterpret_cast<u32x4 *>(tile + slot[j] + 8) = dequant8(c.z, c.w, zero, d2);
            } else {
                // byte i of a block's 16: element i in the low nibble, element 16 + i in the high one
                const half2_t zero = {(_Float16)1032.0f, (_Float16)1032.0f};   // 1024 + 8
                const uint32_t m = 0x0F0F0F0Fu;
                *reinterpret_cast<u32x4 *>(tile + slot[j]) = dequant8(c.x & m, c.y & m, zero, d2);
                *reinterpret_cast<u32x4 *>(tile + slot[j] + 8) = dequant8(c.z & m, c.w & m, zero, d2);
                *reinterpret_cast<u32x4 *>(tile + slot[j] + 16) = dequant8((c.x >> 4) & m, (c.y >> 4) & m, zero, d2);
                *reinterpret_cast<u32x4 *>(tile + slot[j] + 24) = dequant8((c.z >> 4) & m, (c.w >> 4) & m, zero, d2);
            }
        }
    };
    static_assert(64 % CPR == 0, "a lane's chunk of a row is the same in every load of a tile");
    u32x4 new_k_chunk = {0u, 0u, 0u, 0u};
    if constexpr (ROPE) {
        if (new_pos >= 0) new_k_chunk = rope_chunk<D>(p.k_new + new_row, cos_row, sin_row, lane % CPR);
    }
    auto fetch = [&](const char *base0, const char *fresh, int t, u32x4 (&dst)[NLD], bool rotate = false) {
        const int t0 = t * kTile;
        const char *base = base0 + (int64_t)t0 * p.kv_stride_t;
        if (t0 + kTile <= T && !(new_pos >= t0 && new_pos < t0 + kTile)) {
#pragma unroll
            for (int j = 0; j < NLD; j++) dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + g_off[j]));
        } else {   // the sequence's last tile (rows past the end repeat the last token, masked below) or the new token's
#pragma unroll
            for (int j = 0; j < NLD; j++) {
                const int c = j * 64 + lane, row = min(c / CPR, T - 1 - t0), dc = c % CPR;
                const char *cache_ptr = base + (uint32_t)row * (uint32_t)p.kv_stride_t + (uint32_t)dc * 16u;
                const bool is_new = t0 + row == new_pos;
                const u32x4 ld = *reinterpret_cast<const u32x4 *>(is_new ? fresh + new_row + dc * 16 : cache_ptr);
                // (ROPE: the lane's chunk of the rotated new key, made once ahead of the loop; dc = lane % CPR for every j.
                // A select after the load, not a branch around it: with a load that some lanes skip the compiler can no
                // longer count what is in flight and every wait of the loop becomes a wait for everything.)
                if constexpr (ROPE) {
                    const bool take = rotate && is_new;
                    dst[j] = u32x4{take ? new_k_chunk.x : ld.x, take ? new_k_chunk.y : ld.y, take ? new_k_chunk.z : ld.z, take ? new_k_chunk.w : ld.w};
                } else {
                    dst[j] = ld;
                }
            }
        }
    };

    // Q^T fragments: row (head) = lane % 32, features 16*ks + 8*hb .. +8 (16-wide: lane % 16, 32*ks + 8*(lane/16) .. +8)
    constexpr int NQF = W16 ? D / 32 : KS;
    half8_t qf[NQF];
    // ROPE: the query's features and their cos / sin are asked for AHEAD of the first tile (the vector-memory counter
    // returns in order: asked for after it, they would arrive after 16 KiB of K and V and the rotation would sit between
    // the tile's arrival and its first product); the partner of features 32 ks + 8 q4 + i, D/2 further on or back, is
    // this lane's own fragment ks +- NQF/2
    half8_t rc[ROPE ? NQF : 1], rs[ROPE ? NQF : 1];
    if constexpr (ROPE) {
#pragma unroll
        for (int ks = 0; ks < NQF; ks++) {
            qf[ks] = *reinterpret_cast<const half8_t *>(qrow + 32 * ks + 8 * q4);
            rc[ks] = *reinterpret_cast<const half8_t *>(cos_row + (32 * ks + 8 * q4) * 2);
            rs[ks] = *reinterpret_cast<const half8_t *>(sin_row + (32 * ks + 8 * q4) * 2);
        }
    }
    int t = tile_begin + w;
    if (t < tile_end) {
        if constexpr (QUANT) {
            fetch_q(kbase, wk.ksbase, t, kpre, ksc);
            fetch_q(vbase, wk.vsbase, t, vpre, vsc);
        } else {
            fetch(kbase, p.k_new, t, kpre, true);
            fetch(vbase, p.v_new, t, vpre);
        }
    }
    if constexpr (ROPE) {
        half8_t a[NQF], bb[NQF];
#pragma unroll
        for (int ks = 0; ks < NQF; ks++) {
            const bool first = ks < NQF / 2;
            const half8_t y = qf[first ? ks + NQF / 2 : ks - NQF / 2];
            a[ks] = qf[ks] * rc[ks], bb[ks] = (first ? -y : y) * rs[ks];
        }
#pragma unroll
        for (int ks = 0; ks < NQF; ks++) asm volatile("" : "+v"(a[ks]), "+v"(bb[ks]));   // two roundings, not a fused multiply-add
#pragma unroll
        for (int ks = 0; ks < NQF; ks++) qf[ks] = a[ks] + bb[ks];
    } else {
#pragma unroll
        for (int ks = 0; ks < NQF; ks++)
            qf[ks] = *reinterpret_cast<const half8_t *>(W16 ? qrow + 32 * ks + 8 * q4 : qrow + 16 * ks + 8 * hb);
    }
#pragma unroll
    for (int ks = 0; ks < NQF; ks++) asm volatile("" : "+v"(qf[ks]));   // settled here, not at first use inside the loop

    float m_run = -INFINITY, l_run = 0.0f;   // log2 domain, already scaled
    float16_t o[W16 ? 1 : DB];
    float4_t o16[W16 ? D / 16 : 1];
#pragma unroll
    for (int db = 0; db < (W16 ? 1 : DB); db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
#pragma unroll
    for (int fb = 0; fb < (W16 ? D / 16 : 1); fb++) o16[fb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // this lane as a SOURCE of the transposing loads: key row (lane%16)/4 of a group of four, features
    // 16*(lane/16 % 2) + 4*(lane%4) of the 32-feature block (16-wide: token group lane/16, features 4*(lane%4))
    const int vsrc_off = W16 ? (4 * q4 + (l16 >> 2)) * VROW + 4 * (l16 & 3)
                             : (4 * hb + ((lane & 15) >> 2)) * VROW + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    // this lane's mask values: its head's row, tokens 8*rq + 4*hb + 0..3 of the tile
    // (16-wide: tokens 16*mb + 4*(lane/16) + 0..3)
    const char *mask_lane = MASK ? wk.mask + (int64_t)min(hcol, g - 1) * p.mask_stride_h + 8 * (W16 ? q4 : hb) : nullptr;
    // The wave's tiles in order: t, then tn.  Plain: a fixed step.  Skewed: round r of nsplit groups gives split s group
    // nsplit r + s, except that in the rounds r % R == R - 1 an even split takes its odd neighbour's group as well
    // (e = 1) and the odd split none.
    const int tstep = wk.tile_step, R = wk.skew_period, nsp = wk.nsplit, sp = wk.skew_split;
    int sr = 0, se = 0, sj = 0;               // round, extra group, r % R of the tile AFTER t
    auto advance = [&](int from) {
        if (R == 0) return from + tstep;
        if ((sp & 1) == 0) {
            if (se == 0 && sj == R - 1) se = 1;
            else sr++, se = 0, sj = sj + 1 == R ? 0 : sj + 1;
        } else {
            sr++, sj = sj + 1 == R ? 0 : sj + 1;
            if (sj == R - 1) sr++, sj = 0;
        }
        return (nsp * sr + sp + se) * kWaves + w;
    };
    int tn = advance(t);
    for (; t < tile_end; t = tn, tn = advance(tn)) {
        const int t0 = t * kTile;
        const bool more = tn < tile_end;
        constexpr int NMK = W16 ? 2 : 4;          // groups of 4 consecutive tokens this lane owns in a tile
        constexpr int kMkStep = W16 ? 16 : 8;     // tokens between them
        half4_t mk[MASK ? NMK : 1];
        if constexpr (MASK) {   // asked for before the products with K, used after them
            const char *mp = mask_lane + (int64_t)t0 * 2;
            if (t0 + kTile <= T) {
#pragma unroll
                for (int rq = 0; rq < NMK; rq++) mk[rq] = *reinterpret_cast<const half4_t *>(mp + 2 * kMkStep * rq);
            } else {   // the row ends inside this tile
#pragma unroll
                for (int rq = 0; rq < NMK; rq++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int tok = t0 + kMkStep * rq + 4 * (W16 ? q4 : hb) + i;
                        mk[rq][i] = tok < T ? *reinterpret_cast<const _Float16 *>(mp + 2 * kMkStep * rq + 2 * i) : (_Float16)0.0f;
                    }
            }
        }
        // ---- K tile -> LDS, the next tile's K into flight ----------------------------------------------
        if constexpr (QUANT) {
            stash_q(kpre, ksc, k_slot);
            if (more) fetch_q(kbase, wk.ksbase, tn, kpre, ksc);
        } else {
#pragma unroll
            for (int j = 0; j < NLD; j++) *reinterpret_cast<u32x4 *>(tile + k_slot[j]) = kpre[j];
            if (more) fetch(kbase, p.k_new, tn, kpre, true);
        }
        half8_t pf16;
        if constexpr (W16) {
            // ---- S^T = K Q^T: two blocks of 16 tokens x 16 heads --------------------------------------------
            float4_t s16[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
            const _Float16 *kt16 = tile + l16 * KROW + 8 * q4;
#pragma unroll
            for (int ks = 0; ks < D / 32; ks++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++) {
                    const half8_t kf = *reinterpret_cast<const half8_t *>(kt16 + 16 * mb * KROW + 32 * ks);
                    s16[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[ks], s16[mb], 0, 0, 0);
                }
            // ---- online softmax of this lane's head over its 8 tokens: t0 + 16*mb + 4*(lane/16) + r ---------
            float tmax = -INFINITY;
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int tok = t0 + 16 * mb + 4 * q4 + r;
                    s16[mb][r] = (t0 + kTile <= T || tok < T) ? s16[mb][r] * p.scale_log2 : -INFINITY;
                    if constexpr (MASK) s16[mb][r] = __builtin_fmaf((float)mk[mb][r], 1.4426950408889634f, s16[mb][r]);
                    tmax = fmaxf(tmax, s16[mb][r]);
                }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const float m_new = fmaxf(m_run, tmax);   // finite without a mask: every tile holds at least one valid token
            const float m_ref16 = (MASK && m_new == -INFINITY) ? 0.0f : m_new;   // masked out entirely with -inf: no NaN
            float psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float pv = fast_exp2(s16[i >> 2][i & 3] - m_ref16);
                psum += pv;
                pf16[i] = (_Float16)pv;
            }
            const bool moved = m_new != m_run;
            const float alpha = fast_exp2(m_run - m_ref16);
            l_run = l_run * alpha + psum;
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
                for (int fb = 0; fb < D / 16; fb++) o16[fb] *= alpha;
            }
        }
        // ---- S^T = K Q^T: 32 tokens x 32 rows ------------------------------------------------------------
        half8_t pf[2];
        if constexpr (!W16) {
        float16_t s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
        const _Float16 *kt = tile + l32 * KROW + 8 * hb;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const half8_t kf = *reinterpret_cast<const half8_t *>(kt + 16 * ks);
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s, 0, 0, 0);
        }
        // ---- online softmax of this lane's head over its 16 tokens: token = t0 + 8*(r/4) + 4*hb + r%4 ----
        float tmax = -INFINITY;
        if (QUANT && t0 + kTile <= T) {   // (the f16 instantiation has no register to spare for a second copy of this)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                s[r] *= p.scale_log2;
                tmax = fmaxf(tmax, s[r]);
            }
        } else {   // possibly the sequence's last tile: tokens past its end do not count
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int tok = t0 + 8 * (r >> 2) + 4 * hb + (r & 3);
                s[r] = (t0 + kTile <= T || tok < T) ? s[r] * p.scale_log2 : -INFINITY;
                if constexpr (MASK) s[r] = __builtin_fmaf((float)mk[r >> 2][r & 3], 1.4426950408889634f, s[r]);
                tmax = fmaxf(tmax, s[r]);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);   // finite without a mask: every tile holds at least one valid token
        // a tile (so far: a row) masked out entirely with -inf must leave the state untouched, not NaN
        const float m_ref = (MASK && m_new == -INFINITY) ? 0.0f : m_new;
        float psum = 0.0f;
#pragma unroll
        for (int st = 0; st < 2; st++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float pv = fast_exp2(s[8 * st + i] - m_ref);
                psum += pv;
                pf[st][i] = (_Float16)pv;
            }
        const bool moved = m_new != m_run;
        const float alpha = fast_exp2(m_run - m_ref);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        }
        }
        // ---- V tile -> the same LDS tile (every K fragment has been consumed), next V into flight ------
        if constexpr (QUANT) {
            stash_q(vpre, vsc, v_slot);
            if (more) fetch_q(vbase, wk.vsbase, tn, vpre, vsc);
        } else {
#pragma unroll
            for (int j = 0; j < NLD; j++) *reinterpret_cast<u32x4 *>(tile + v_slot[j]) = vpre[j];
            if (more) fetch(vbase, p.v_new, tn, vpre);
        }
        // ---- O^T += V^T P^T ---------------------------------------------------------------------------------
        const _Float16 *vsrc = tile + vsrc_off;
        if constexpr (W16) {
#pragma unroll
            for (int fb = 0; fb < D / 16; fb++) {
                const half4_t lo = lds_read_tr16(vsrc + 16 * fb);               // tokens 4*(lane/16) + 0..3
                const half4_t hi = lds_read_tr16(vsrc + 16 * VROW + 16 * fb);   // tokens 16 + 4*(lane/16) + 0..3
                const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                o16[fb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf16, o16[fb], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    const half4_t lo = lds_read_tr16(vsrc + (16 * st) * VROW + 32 * db);      // tokens 16st + 4hb + 0..3
                    const half4_t hi = lds_read_tr16(vsrc + (16 * st + 8) * VROW + 32 * db);  // tokens 16st + 8 + 4hb + 0..3
                    const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[st], o[db], 0, 0, 0);
                }
        }
    }
    if constexpr (W16) l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);

    // ---- merge the 4 waves through LDS (the K/V tiles are dead) --------------------------------------------
    __syncthreads();
    float *comb = reinterpret_cast<float *>(lds_raw);   // [kWaves][GP*D + 2*GP]
    if constexpr (W16) {
        if (l16 < GP) {
            float *cw = comb + w * kCombStride;
#pragma unroll
            for (int fb = 0; fb < D / 16; fb++) *reinterpret_cast<float4_t *>(cw + l16 * D + 16 * fb + 4 * q4) = o16[fb];
            if (q4 == 0) {
                cw[GP * D + l16] = m_run;
                cw[GP * D + GP + l16] = l_run;
            }
        }
    } else if (l32 < GP) {
        float *cw = comb + w * kCombStride;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                float4_t f4 = {o[db][4 * rq], o[db][4 * rq + 1], o[db][4 * rq + 2], o[db][4 * rq + 3]};
                *reinterpret_cast<float4_t *>(cw + l32 * D + 32 * db + 8 * rq + 4 * hb) = f4;
            }
        if (hb == 0) {
            cw[GP * D + l32] = m_run;
            cw[GP * D + GP + l32] = l_run;
        }
    }
    wave_records_to_output<D, GP>(p, wk, lds_raw, head0, g, tid);
}

// Transposing 64-bit LDS load of 8-bit elements: in each block of 16 lanes, lane i receives byte i%8 of the eight
// 8-byte rows addressed by lanes i/8, i/8 + 2, ..., i/8 + 14 of the block, in that order.
__device__ __forceinline__ void lds_read_tr8(const unsigned char *lds_ptr, uint32_t &w0, uint32_t &w1) {
    typedef int int2_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) int2_t *lds_v2_ptr;
    const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2_ptr)(uintptr_t)(uint32_t)(uintptr_t)lds_ptr);
    w0 = (uint32_t)r[0], w1 = (uint32_t)r[1];
}
// eight unsigned bytes as the eight halves 1024 + b (exact integers in f16)
__device__ __forceinline__ half8_t magic8(uint32_t w0, uint32_t w1) {
    u32x4 r;
    r.x = perm(0x64646464u, w0, 0x04010400u), r.y = perm(0x64646464u, w0, 0x04030402u);
    r.z = perm(0x64646464u, w1, 0x04010400u), r.w = perm(0x64646464u, w1, 0x04030402u);
    return __builtin_bit_cast(half8_t, r);
}

// Block-quantised caches (Q8_0 / Q4_0, head_dim 128, up to 16 heads per kv head) without dequantising any element.
// The contraction of v_mfma_f32_16x16x32_f16 is 32 features deep, exactly one quantisation block, so the raw codes go
// into the matrix cores as the exact f16 integers 1024 + u (one v_perm per two codes puts the byte under the exponent
// byte 0x64; Q4_0's high nibbles stay where they are, as 16 u, against query features divided by 16) and the block
// scales are applied outside the products:
//   scores:  S[t, h] = sum_blk d_k[t, blk] * (acc_blk[t, h] - bias[h, blk]);  the bias, (1024 + zero) * sum of the
//            block's query features, is a constant of the lane's head and rides in as the accumulator's initial value;
//   outputs: O[f, h] = sum_t (u_v[t, f] - zero) * (P[t, h] * d_v[t, blk(f)]): the scale is folded into the probabilities
//            (one packed multiply per block and token pair), and the zero point is taken out once at the end through
//            SP[h, blk] = sum_t P[t, h] * d_v[t, blk], accumulated beside the outputs.
// The products are exact in f32 where the reference rounds every dequantised element to f16 first (q4_0.rs:82-95):
// the two differ by at most half an f16 unit per element, inside the tolerance of the path.
// Per wave and 32-token tile: code rows global -> registers (one tile ahead, non-temporal 128-bit loads) -> raw bytes in
// a wave-private LDS tile (consecutive lanes write consecutive 16-byte slots) -> K fragments by 8-byte (Q4_0: 4-byte)
// reads, V^T fragments by transposing byte reads; the f16 block scales of the tile (256 bytes per tensor) go through
// LDS too.
// A decode step's new token on a block-quantised cache (the fused append): quantised once, by the wave whose tiles
// include the sequence's last one, exactly as the append kernel would (quant_block.h), written to the cache planes and
// kept in `lds_new` (K codes, V codes, the K scales, the V scales), from where that wave's tile takes the row -- no other
// wave of the launch reads it.  Lanes 0..3 take the four K blocks of the row, lanes 4..7 the V blocks.
template <int FMT, bool ROPE = false>
__device__ __forceinline__ void quantise_new_token(const DecodeDev &p, const MfmaWork &wk, int lane, unsigned char *lds_new) {
    constexpr bool Q8 = FMT == TROCM_Q8_0;
    constexpr int D = 128, RB = Q8 ? D : D / 2, BB = Q8 ? 32 : 16, SROW = (D / 32) * 2;
    if (lane < 8) {
        const int blk = lane & 3;
        const bool is_v = lane >= 4;
        const __half *src = reinterpret_cast<const __half *>(is_v ? p.v_new : p.k_new) + ((int64_t)wk.seq * p.Hkv + wk.kvh) * D + 32 * blk;
        float v[32];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint4 x = reinterpret_cast<const uint4 *>(src)[i];
            if constexpr (ROPE) {   // the key is rotated (ApplyRope, rounded to f16) before it is quantised
                if (!is_v) {
                    const char *cs = p.rope_cos + (int64_t)wk.seq * p.rope_stride_b, *sn = p.rope_sin + (int64_t)wk.seq * p.rope_stride_b;
                    x = __builtin_bit_cast(uint4, rope_piece128<8>(reinterpret_cast<const _Float16 *>(src) - 32 * blk, cs, sn, 32 * blk + 8 * i));
                }
            }
            const __half *e = reinterpret_cast<const __half *>(&x);
#pragma unroll
            for (int j = 0; j < 8; j++) v[8 * i + j] = __half2float(e[j]);
        }
        unsigned char *codes_lds = lds_new + (is_v ? RB : 0) + blk * BB;
        char *codes_mem = const_cast<char *>(is_v ? wk.vbase : wk.kbase) + (int64_t)wk.new_pos * RB + blk * BB;
        uint16_t d;
        if constexpr (Q8) {
            uint32_t c[8];
            d = quant_q8(v, c);
            constexpr uint32_t x = 0x80808080u;   // the plane holds code + 128
            const u32x4 lo4 = {c[0] ^ x, c[1] ^ x, c[2] ^ x, c[3] ^ x}, hi4 = {c[4] ^ x, c[5] ^ x, c[6] ^ x, c[7] ^ x};
            reinterpret_cast<u32x4 *>(codes_lds)[0] = lo4, reinterpret_cast<u32x4 *>(codes_lds)[1] = hi4;
            reinterpret_cast<u32x4 *>(codes_mem)[0] = lo4, reinterpret_cast<u32x4 *>(codes_mem)[1] = hi4;
        } else {
            uint32_t c[4];
            d = quant_q4(v, c);
            const u32x4 c4 = {c[0], c[1], c[2], c[3]};
            *reinterpret_cast<u32x4 *>(codes_lds) = c4;
            *reinterpret_cast<u32x4 *>(codes_mem) = c4;
        }
        reinterpret_cast<uint16_t *>(lds_new + 2 * RB)[lane] = d;   // K scales 0..3, V scales 4..7
        *reinterpret_cast<uint16_t *>(const_cast<char *>(is_v ? wk.vsbase : wk.ksbase) + (int64_t)wk.new_pos * SROW + blk * 2) = d;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the wave's other lanes read the row back from LDS
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
constexpr int kNewTokenLdsBytes = 2 * 128 + 16;   // two rows of codes (Q8_0: 128 bytes each) and eight scales

template <int GP, int FMT, int PF>
__device__ __forceinline__ void decode_mfma_qblock_body(const DecodeDev &p, const MfmaWork &wk) {
    static_assert(GP <= 16, "the 16-wide layout: at most 16 heads");
    static_assert(FMT == TROCM_Q8_0 || FMT == TROCM_Q4_0, "block-quantised caches only");
    constexpr int D = 128;
    constexpr bool Q8 = FMT == TROCM_Q8_0;
    constexpr int NB = D / 32;                 // blocks per token row
    constexpr int RB = Q8 ? D : D / 2;         // code bytes per token row
    constexpr int NLD = kTile * RB / 1024;     // 128-bit loads per lane, tile and tensor: 4 / 2
    constexpr int CPR = RB / 16;               // 16-byte chunks per row: 8 / 4
    constexpr int SROW = NB * 2;               // bytes of block scales per row
    constexpr int kCodeBytes = kTile * RB;     // one tensor's tile in LDS
    constexpr int kScaleBytes = kTile * SROW;
    constexpr int kWaveBytes = 2 * kCodeBytes + 2 * kScaleBytes + kNewTokenLdsBytes;
    constexpr int kCombStride = GP * D + 2 * GP;
    constexpr int kLdsBytes = kWaves * (kWaveBytes > kCombStride * 4 ? kWaveBytes : kCombStride * 4);
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLdsBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, q4 = lane >> 4;
    const int kvh = wk.kvh, b = wk.seq;
    const int g = p.g_real;
    unsigned char *lds_k = lds_raw + w * kWaveBytes, *lds_v = lds_k + kCodeBytes;
    unsigned char *lds_ks = lds_v + kCodeBytes, *lds_vs = lds_ks + kScaleBytes;

    const int64_t head0 = (int64_t)b * p.Hq + (int64_t)kvh * g;
    const _Float16 *qrow = reinterpret_cast<const _Float16 *>(p.q) + (head0 + min(l16, g - 1)) * D;
    const int T = wk.T;
    const int tile_begin = wk.tile_begin, tile_end = wk.tile_end;

    // one tile ahead in registers: NLD chunks of 16 code bytes (chunk j*64 + lane of the tile, rows are dense) and,
    // in lanes 0..31, the 8 bytes of block scales of token `lane`
    // (PF tiles ahead: a wave's tile of Q4_0 codes is 2 KiB per tensor, and 2048 waves with one tile each in flight do
    // not cover the memory latency at full bandwidth)
    u32x4 kpre[PF][NLD], vpre[PF][NLD];
    u32x2 kspre[PF], vspre[PF];
    // (a fused append's new token is the sequence's last: its tile takes the row from lds_new, see quantise_new_token)
    const int new_pos = wk.new_pos;
    unsigned char *lds_new = lds_raw + w * kWaveBytes + 2 * kCodeBytes + 2 * kScaleBytes;
    auto fetch = [&](const char *base0, const char *sbase0, int which, int t, u32x4 (&dst)[NLD], u32x2 &sc) {
        const int t0 = t * kTile;
        const char *base = base0 + (int64_t)t0 * RB;
        const char *sbase = sbase0 + (int64_t)t0 * SROW;
        if (t0 + kTile <= T && !(new_pos >= t0 && new_pos < t0 + kTile)) {
#pragma unroll
            for (int j = 0; j < NLD; j++)
                dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + (j * 64 + lane) * 16));
            if (lane < kTile) sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(sbase + lane * SROW));
        } else {   // rows past the end of the sequence repeat its last token (their scores are masked below)
            const int last = T - 1 - t0;
#pragma unroll
            for (int j = 0; j < NLD; j++) {
                const int c = j * 64 + lane, row = min(c / CPR, last), dc = c % CPR;
                if (t0 + row == new_pos) dst[j] = *reinterpret_cast<const u32x4 *>(lds_new + which * RB + dc * 16);
                else dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + row * RB + dc * 16));
            }
            if (lane < kTile) {
                const int row = min(lane, last);
                if (t0 + row == new_pos) sc = *reinterpret_cast<const u32x2 *>(lds_new + 2 * RB + which * 8);
                else sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(sbase + row * SROW));
            }
        }
    };
    // Where this lane's chunks go in the LDS tiles.  The 16-byte chunks of a row are permuted (xor with a key of the row)
    // so that the fragment reads below, which walk down the rows at a fixed place in the row, spread over the banks: the
    // K tile is read 16 consecutive tokens at a time (key: the token's low bits), the V tile 4 + 4 tokens 16 apart (key:
    // low bits and bit 4 of the token).  A row stays one contiguous 128- or 64-byte run, so the writes stay conflict-free.
    auto key_k = [](int row) { return Q8 ? (row & 7) : ((row >> 1) & 3); };
    auto key_v = [](int row) { return Q8 ? ((row & 3) | (((row >> 4) & 1) << 2)) : (((row >> 1) & 1) | (((row >> 4) & 1) << 1)); };
    uint32_t k_slot[NLD], v_slot[NLD];
#pragma unroll
    for (int j = 0; j < NLD; j++) {
        const int c = j * 64 + lane, row = c / CPR, dc = c % CPR;
        k_slot[j] = row * RB + 16 * (dc ^ key_k(row));
        v_slot[j] = row * RB + 16 * (dc ^ key_v(row));
    }
    const int tstep = wk.tile_step;
    int t = tile_begin + w;
    if (new_pos >= 0) {   // (wave-uniform) the wave whose tiles include the new token's quantises and stores it
        const int nt = new_pos / kTile;
        if (nt >= t && nt < tile_end && (nt - t) % tstep == 0) quantise_new_token<FMT>(p, wk, lane, lds_new);
    }
#pragma unroll
    for (int st = 0; st < PF; st++) {
        kspre[st] = vspre[st] = u32x2{0u, 0u};
        if (t + st * tstep < tile_end) {
            fetch(wk.kbase, wk.ksbase, 0, t + st * tstep, kpre[st], kspre[st]);
            fetch(wk.vbase, wk.vsbase, 1, t + st * tstep, vpre[st], vspre[st]);
        }
    }

    // Q^T fragments of this lane's head, one per block: the 8 features that lane group q4 contributes.
    //   Q8_0: features 32 blk + 8 q4 + 0..7
    //   Q4_0: features 32 blk + 4 q4 + 0..3 (low nibbles) and 32 blk + 16 + 4 q4 + 0..3 (high nibbles: the codes arrive
    //         as 16 u, so these features are divided by 16 -- exact but for subnormal results)
    half8_t qf[NB];
    float bias[NB];   // (1024 + zero) * (what the products add up for a block of all-zero-point codes), negated
#pragma unroll
    for (int blk = 0; blk < NB; blk++) {
        float part;
        if constexpr (Q8) {
            qf[blk] = *reinterpret_cast<const half8_t *>(qrow + 32 * blk + 8 * q4);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) sum += (float)qf[blk][i];
            part = 1152.0f * sum;   // the plane holds code + 128, under 1024
        } else {
            const half4_t lo = *reinterpret_cast<const half4_t *>(qrow + 32 * blk + 4 * q4);
            const half4_t hi = *reinterpret_cast<const half4_t *>(qrow + 32 * blk + 16 + 4 * q4);
            float s_lo = 0.0f, s_hi = 0.0f, s_hi16 = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const _Float16 h16 = hi[i] * (_Float16)0.0625f;
                qf[blk][i] = lo[i], qf[blk][4 + i] = h16;
                s_lo += (float)lo[i], s_hi16 += (float)h16, s_hi += 16.0f * (float)h16;
            }
            part = 1024.0f * (s_lo + s_hi16) + 8.0f * (s_lo + s_hi);
        }
        part += __shfl_xor(part, 16, 64);
        part += __shfl_xor(part, 32, 64);
        bias[blk] = -part;
    }
#pragma unroll
    for (int blk = 0; blk < NB; blk++) asm volatile("" : "+v"(qf[blk]));   // settled here, not at first use inside the loop

    float m_run = -INFINITY, l_run = 0.0f;   // log2 domain, already scaled
    float4_t o16[D / 16];
    float sp[NB];
#pragma unroll
    for (int fb = 0; fb < D / 16; fb++) o16[fb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int blk = 0; blk < NB; blk++) sp[blk] = 0.0f;

    // K fragment of this lane: token 16 mb + l16 (its key does not depend on mb), the bytes of block blk that lane group
    // q4 contributes: Q8_0 chunk 2 blk + q4 / 2, half q4 % 2; Q4_0 chunk blk, word q4
    uint32_t k_frag[NB];
#pragma unroll
    for (int blk = 0; blk < NB; blk++)
        k_frag[blk] = Q8 ? l16 * RB + 16 * ((2 * blk + (q4 >> 1)) ^ key_k(l16)) + 8 * (q4 & 1) : l16 * RB + 16 * (blk ^ key_k(l16)) + 4 * q4;
    // V^T fragments: this lane as a SOURCE of the transposing reads addresses token (4 q4 + k, or 16 + 4 q4 + k - 4: the
    // order of the probabilities in the B fragment), bytes 8 (l16 % 2) .. + 8 of a 16-byte group; k = l16 / 2
    const int vk = l16 >> 1, v_tok = vk < 4 ? 4 * q4 + vk : 12 + 4 * q4 + vk;
    const unsigned char *v_row = lds_v + v_tok * RB + 8 * (l16 & 1);
    const uint32_t v_key16 = 16 * key_v(v_tok);   // (16 c) ^ v_key16 = 16 (c ^ key)
    // block scales of this lane's tokens 16 mb + 4 q4 + 0..3: 32 contiguous bytes per mb
    const unsigned char *ks_frag = lds_ks + 4 * q4 * SROW, *vs_frag = lds_vs + 4 * q4 * SROW;
    const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};

    const float c_log2 = p.scale_log2;   // > 0 (checked on the host): the maximum is taken before scaling
    // one tile, whose codes wait in stage ST of the prefetch registers
    auto do_tile = [&](auto stage_tag, int t) {
        constexpr int ST = decltype(stage_tag)::value;
        const int t0 = t * kTile;
        const bool more = t + PF * tstep < tile_end;
        // ---- this tile's codes and scales -> LDS, the tile PF steps on into flight --------------------------------
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            *reinterpret_cast<u32x4 *>(lds_k + k_slot[j]) = kpre[ST][j];
            *reinterpret_cast<u32x4 *>(lds_v + v_slot[j]) = vpre[ST][j];
        }
        if (lane < kTile) {
            *reinterpret_cast<u32x2 *>(lds_ks + lane * SROW) = kspre[ST];
            *reinterpret_cast<u32x2 *>(lds_vs + lane * SROW) = vspre[ST];
        }
        if (more) {
            fetch(wk.kbase, wk.ksbase, 0, t + PF * tstep, kpre[ST], kspre[ST]);
            fetch(wk.vbase, wk.vsbase, 1, t + PF * tstep, vpre[ST], vspre[ST]);
        }
        // ---- per block: codes x query features, the bias riding in the accumulator -------------------------------
        float4_t acc[2][NB];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int blk = 0; blk < NB; blk++) {
                half8_t kf;
                if constexpr (Q8) {
                    const u32x2 c = *reinterpret_cast<const u32x2 *>(lds_k + k_frag[blk] + 16 * mb * RB);
                    kf = magic8(c.x, c.y);   // (the plane holds code + 128)
                } else {
                    const uint32_t c = *reinterpret_cast<const uint32_t *>(lds_k + k_frag[blk] + 16 * mb * RB);
                    kf = magic8(c & 0x0F0F0F0Fu, c & 0xF0F0F0F0u);
                }
                const float4_t c0 = {bias[blk], bias[blk], bias[blk], bias[blk]};
                acc[mb][blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[blk], c0, 0, 0, 0);
            }
        // ---- scores (before the softmax scale): the block scales of this lane's tokens 16 mb + 4 q4 + r ---------------
        float sc8[8];
        float tmax = -INFINITY;
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
            const u32x4 d01 = *reinterpret_cast<const u32x4 *>(ks_frag + 16 * mb * SROW);        // tokens r = 0, 1: (d0 d1)(d2 d3) each
            const u32x4 d23 = *reinterpret_cast<const u32x4 *>(ks_frag + 16 * mb * SROW + 16);   // tokens r = 2, 3
            const uint32_t dw[4][2] = {{d01.x, d01.y}, {d01.z, d01.w}, {d23.x, d23.y}, {d23.z, d23.w}};
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const half2_t da = as_half2(dw[r][0]), db = as_half2(dw[r][1]);
                float sv = __builtin_fmaf((float)da[0], acc[mb][0][r], 0.0f);
                sv = __builtin_fmaf((float)da[1], acc[mb][1][r], sv);
                sv = __builtin_fmaf((float)db[0], acc[mb][2][r], sv);
                sv = __builtin_fmaf((float)db[1], acc[mb][3][r], sv);
                sc8[4 * mb + r] = sv;
            }
        }
        if (t0 + kTile > T) {   // the sequence's last tile: tokens past its end do not count
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (t0 + 16 * (i >> 2) + 4 * q4 + (i & 3) >= T) sc8[i] = -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 8; i++) tmax = fmaxf(tmax, sc8[i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax * c_log2);   // finite: every tile holds at least one valid token
        float psum = 0.0f;
        half2_t pf[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float p0 = fast_exp2(__builtin_fmaf(sc8[2 * i], c_log2, -m_new)), p1 = fast_exp2(__builtin_fmaf(sc8[2 * i + 1], c_log2, -m_new));
            psum += p0 + p1;
            pf[i] = half2_t{(_Float16)p0, (_Float16)p1};
        }
        const bool moved = m_new != m_run;
        const float alpha = fast_exp2(m_run - m_new);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int fb = 0; fb < D / 16; fb++) o16[fb] *= alpha;
#pragma unroll
            for (int blk = 0; blk < NB; blk++) sp[blk] *= alpha;
        }
        // ---- probabilities times the V block scales of their tokens, per block -----------------------------------------
        // pf[i] holds tokens (4 q4 + 2i, + 1) for i < 2 and (16 + 4 q4 + 2(i - 2), + 1) for i >= 2
        half8_t pb[NB];
        {
            const u32x4 e0 = *reinterpret_cast<const u32x4 *>(vs_frag);                       // mb 0: tokens r = 0, 1
            const u32x4 e1 = *reinterpret_cast<const u32x4 *>(vs_frag + 16);                  //       r = 2, 3
            const u32x4 e2 = *reinterpret_cast<const u32x4 *>(vs_frag + 16 * SROW);           // mb 1: r = 0, 1
            const u32x4 e3 = *reinterpret_cast<const u32x4 *>(vs_frag + 16 * SROW + 16);      //       r = 2, 3
            const u32x4 ev[4] = {e0, e1, e2, e3};   // ev[i] = rows of the token pair of pf[i]: (x y) first token, (z w) second
#pragma unroll
            for (int blk = 0; blk < NB; blk++) {
                u32x4 pw;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t first = (blk < 2) ? ev[i].x : ev[i].y, second = (blk < 2) ? ev[i].z : ev[i].w;
                    const half2_t dd = as_half2(perm(second, first, (blk & 1) ? 0x07060302u : 0x05040100u));
                    const half2_t pp = pf[i] * dd;
                    sp[blk] = __builtin_amdgcn_fdot2(pp, ones, sp[blk], false);
                    pw[i] = __builtin_bit_cast(uint32_t, pp);
                }
                pb[blk] = __builtin_bit_cast(half8_t, pw);
            }
        }
        // ---- O^T += codes^T x scaled probabilities -----------------------------------------------------------------------
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            if constexpr (Q8) {
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    uint32_t w0, w1;
                    lds_read_tr8(v_row + ((32 * blk + 16 * hf) ^ v_key16), w0, w1);
                    const half8_t vf = magic8(w0, w1);
                    o16[2 * blk + hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pb[blk], o16[2 * blk + hf], 0, 0, 0);
                }
            } else {
                uint32_t w0, w1;   // byte l16 of the block's 16: feature l16 in the low nibble, 16 + l16 in the high one
                lds_read_tr8(v_row + ((16 * blk) ^ v_key16), w0, w1);
                const half8_t vlo = magic8(w0 & 0x0F0F0F0Fu, w1 & 0x0F0F0F0Fu);
                const half8_t vhi = magic8(w0 & 0xF0F0F0F0u, w1 & 0xF0F0F0F0u);
                o16[2 * blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vlo, pb[blk], o16[2 * blk], 0, 0, 0);
                o16[2 * blk + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vhi, pb[blk], o16[2 * blk + 1], 0, 0, 0);
            }
        }
    };
    static_assert(PF <= 4, "stages are written out");
    while (t < tile_end) {
        do_tile(std::integral_constant<int, 0>{}, t);
        t += tstep;
        if constexpr (PF > 1) {
            if (t < tile_end) do_tile(std::integral_constant<int, 1>{}, t), t += tstep;
        }
        if constexpr (PF > 2) {
            if (t < tile_end) do_tile(std::integral_constant<int, 2>{}, t), t += tstep;
        }
        if constexpr (PF > 3) {
            if (t < tile_end) do_tile(std::integral_constant<int, 3>{}, t), t += tstep;
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    // the zero points: O[f, h] -= (1024 + zero) * SP[h, blk(f)] (Q4_0's high features arrived 16 times too large)
#pragma unroll
    for (int blk = 0; blk < NB; blk++) {
        float s_all = sp[blk];
        s_all += __shfl_xor(s_all, 16, 64);
        s_all += __shfl_xor(s_all, 32, 64);
        if constexpr (Q8) {
            o16[2 * blk] -= 1152.0f * s_all;
            o16[2 * blk + 1] -= 1152.0f * s_all;
        } else {
            o16[2 * blk] -= 1032.0f * s_all;
            o16[2 * blk + 1] = o16[2 * blk + 1] * 0.0625f - 72.0f * s_all;
        }
    }

    // ---- merge the 4 waves through LDS (the tiles are dead) ------------------------------------------------------------
    __syncthreads();
    float *comb = reinterpret_cast<float *>(lds_raw);   // [kWaves][GP*D + 2*GP]
    if (l16 < GP) {
        float *cw = comb + w * kCombStride;
#pragma unroll
        for (int fb = 0; fb < D / 16; fb++) *reinterpret_cast<float4_t *>(cw + l16 * D + 16 * fb + 4 * q4) = o16[fb];
        if (q4 == 0) {
            cw[GP * D + l16] = m_run;
            cw[GP * D + GP + l16] = l_run;
        }
    }
    wave_records_to_output<D, GP>(p, wk, lds_raw, head0, g, tid);
}

// Eight nibbles of a word as eight halves with one shift and four and-or: (w & 0x000F000F) | 0x64006400 is the pair
// (1024 + n0, 1024 + n4), (w & 0x00F000F0) | 0x64006400 the pair (1024 + 16 n1, 1024 + 16 n5), and w >> 8 brings n2, n6
// and n3, n7 to the same places.  For a word of four Q4_0 bytes b0..b3 (low nibble = one element, high nibble = another):
// halves (lo0, lo2), 16 (hi0, hi2), (lo1, lo3), 16 (hi1, hi3).  The three constants come in vector registers (laundered
// through an empty asm once per kernel): as literals, v_and_or_b32 cannot take two of them and the compiler emits an and
// and an or instead.
struct NibbleConsts {
    uint32_t lo, hi, magic;
};
__device__ __forceinline__ NibbleConsts nibble_consts() {
    NibbleConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u};
    asm volatile("" : "+v"(c.lo), "+v"(c.hi), "+v"(c.magic));
    return c;
}
__device__ __forceinline__ void nibbles8(const NibbleConsts &c, uint32_t w, uint32_t &lo02, uint32_t &hi02, uint32_t &lo13, uint32_t &hi13) {
    const uint32_t t = w >> 8;
    lo02 = (w & c.lo) | c.magic, hi02 = (w & c.hi) | c.magic;
    lo13 = (t & c.lo) | c.magic, hi13 = (t & c.hi) | c.magic;
}

// The same block-scaling arithmetic for up to 4 heads per kv head, with no idle column in the 16-wide tiles: column
// c = 4 blk + h of a score tile stands for (quantisation block blk, head h).  The 32-deep contraction of one
// v_mfma_f32_16x16x32_f16 takes 8 features of EACH of a token's four blocks (lane group q4 feeds block q4), and the
// query operand is block diagonal: column (blk, h) holds head h's features of block blk in the lanes of group blk and
// zeros elsewhere.  Four such products (one per 8-feature slice j of the blocks) leave, in column (blk, h), the sum
// over block blk alone -- what the block-scaling body keeps in four accumulators -- so that
//   * a lane scales its four tokens' sums by ONE block's scales (4 multiplications per 16 tokens instead of 16), and the
//     four blocks of a head are added across lanes (two row rotations);
//   * the probabilities times the V block scales are ONE operand for all four blocks (column (blk, h) carries
//     P[t, h] d_v[t, blk]; an output tile of block b is read off the columns (b, h)): 4 packed multiplications and 4
//     dot products per tile where the block-scaling body needs 16 + 16, and no shuffling of scales at all, because
//     the scale tiles are kept transposed in LDS ([block][token]: a lane's four tokens are one 8-byte read).
// Matrix instructions, code unpacking and LDS traffic per tile are those of the block-scaling body.
//
// H = 8 (5..8 heads per kv head): column c = 8 blk' + h stands for (block blk' of a PAIR of blocks, head h).  One product
// then takes 16 features of each of two blocks (lane groups 2 blk', 2 blk' + 1 feed block blk' of the pair), a token's
// four blocks take two sets of products (X = 0: blocks 0, 1; X = 1: blocks 2, 3) into two accumulators, a lane scales
// the sums of two blocks and adds them in place, and one row rotation joins the pair.  The probabilities need one
// operand per set (column (blk', h) carries P[t, h] d_v[t, 2 X + blk']).  Products, unpacking and LDS traffic per tile
// stay what they are for H = 4; 16 vector instructions per tile are added.
//
// RS: the lanes that hold a head's blocks are neighbours (column c = BPC h + blk) and the sum over the blocks is a
// reduce-scatter instead of an all-reduce.  The lanes that feed block blk of a set read token row (l ^ blk) of a
// 16-token half where the others read row l, so register r of lane (h, blk) holds token (r ^ blk) of its group of four.
// H = 4:  y = x0 + swap1(x1),  w = x2 + swap1(x3),  z = y + swap2(w)  (swap1 / swap2: the lane 1 / 2 places across in
// the quad, DPP quad_perm) is, in lane blk, the whole score of token blk: three additions per half instead of eight,
// every register index static; a lane exponentiates TWO scores (one per half) instead of eight.  H = 8:  x0 + swap1(x1)
// and x2 + swap1(x3) are the scores of tokens blk and 2 + blk: two additions per half instead of four, four
// exponentials instead of eight.  The pairs (token j of the first half, of the second) are then handed round with four
// quad broadcasts, which put token j's pair into register j of every lane.
template <int GP, int FMT, int PF, int H = 4, bool RS = false, bool ROPE = false>
__device__ __forceinline__ void decode_mfma_qdiag_body(const DecodeDev &p, const MfmaWork &wk) {

    static_assert(GP == 8, "partial records are 8 rows wide; with H = 4 rows 0..3 are used");
    static_assert(H == 4 || H == 8, "4 or 8 heads across the 16 columns");
    static_assert(FMT == TROCM_Q8_0 || FMT == TROCM_Q4_0, "block-quantised caches only");
    constexpr int D = 128;
    constexpr bool Q8 = FMT == TROCM_Q8_0;
    constexpr int NB = D / 32;                 // blocks per token row
    constexpr int RB = Q8 ? D : D / 2;         // code bytes per token row
    constexpr int NLD = kTile * RB / 1024;     // 128-bit loads per lane, tile and tensor: 4 / 2
    constexpr int CPR = RB / 16;               // 16-byte chunks per row: 8 / 4
    constexpr int SROW = NB * 2;               // bytes of block scales per row
    constexpr int kCodeBytes = kTile * RB;     // one tensor's tile in LDS
    constexpr int kScaleBytes = kTile * SROW;
    constexpr int kWaveBytes = 2 * kCodeBytes + 2 * kScaleBytes + kNewTokenLdsBytes;
    constexpr int kCombStride = GP * D + 2 * GP;
    constexpr int kLdsBytes = kWaves * (kWaveBytes > kCombStride * 4 ? kWaveBytes : kCombStride * 4);
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLdsBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, q4 = lane >> 4;
    constexpr int BPC = 16 / H;                // blocks per product: 4 | 2
    constexpr int LG = 4 / BPC;                // lane groups that feed one block of a product: 1 | 2
    constexpr int NX = NB / BPC;               // sets of products per token: 1 | 2
    constexpr int NJ = 4 / LG;                 // 8-code slices of a block per lane: 4 | 2
    const int blk_c = RS ? l16 % BPC : l16 / H, h_c = RS ? l16 / BPC : l16 % H;  // this lane's column: (block within a set, head)
    const int qb = q4 / LG, qs = q4 % LG;      // as a feeder: block within a set, and which slices of it (qs NJ + j)
    const int kvh = wk.kvh, b = wk.seq;
    const int g = p.g_real;
    unsigned char *lds_k = lds_raw + w * kWaveBytes, *lds_v = lds_k + kCodeBytes;
    unsigned char *lds_ks = lds_v + kCodeBytes, *lds_vs = lds_ks + kScaleBytes;   // scales, transposed: [block][token] f16

    const int64_t head0 = (int64_t)b * p.Hq + (int64_t)kvh * g;
    const _Float16 *qrow = reinterpret_cast<const _Float16 *>(p.q) + (head0 + min(h_c, g - 1)) * D;
    const int T = wk.T;
    const int tile_begin = wk.tile_begin, tile_end = wk.tile_end;

    u32x4 kpre[PF][NLD], vpre[PF][NLD];
    u32x2 kspre[PF], vspre[PF];
    // (a fused append's new token is the sequence's last: its tile takes the row from lds_new, see quantise_new_token)
    const int new_pos = wk.new_pos;
    unsigned char *lds_new = lds_raw + w * kWaveBytes + 2 * kCodeBytes + 2 * kScaleBytes;
    auto fetch = [&](const char *base0, const char *sbase0, int which, int t, u32x4 (&dst)[NLD], u32x2 &sc) {
        const int t0 = t * kTile;
        const char *base = base0 + (int64_t)t0 * RB;
        const char *sbase = sbase0 + (int64_t)t0 * SROW;
        if (t0 + kTile <= T && !(new_pos >= t0 && new_pos < t0 + kTile)) {
#pragma unroll
            for (int j = 0; j < NLD; j++)
                dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + (j * 64 + lane) * 16));
            if (lane < kTile) sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(sbase + lane * SROW));
        } else {   // rows past the end of the sequence repeat its last token (their scores are masked below)
            const int last = T - 1 - t0;
#pragma unroll
            for (int j = 0; j < NLD; j++) {
                const int c = j * 64 + lane, row = min(c / CPR, last), dc = c % CPR;
                if (t0 + row == new_pos) dst[j] = *reinterpret_cast<const u32x4 *>(lds_new + which * RB + dc * 16);
                else dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + row * RB + dc * 16));
            }
            if (lane < kTile) {
                const int row = min(lane, last);
                if (t0 + row == new_pos) sc = *reinterpret_cast<const u32x2 *>(lds_new + 2 * RB + which * 8);
                else sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(sbase + row * SROW));
            }
        }
    };
    // code tiles in LDS exactly as in the block-scaling body (16-byte chunks of a row permuted by a key of the row)
    auto key_k = [](int row) { return Q8 ? (row & 7) : ((row >> 1) & 3); };
    auto key_v = [](int row) { return Q8 ? ((row & 3) | (((row >> 4) & 1) << 2)) : (((row >> 1) & 1) | (((row >> 4) & 1) << 1)); };
    uint32_t k_slot[NLD], v_slot[NLD];
#pragma unroll
    for (int j = 0; j < NLD; j++) {
        const int c = j * 64 + lane, row = c / CPR, dc = c % CPR;
        k_slot[j] = row * RB + 16 * (dc ^ key_k(row));
        v_slot[j] = row * RB + 16 * (dc ^ key_v(row));
    }
    const int tstep = wk.tile_step;
    int t = tile_begin + w;
    auto new_token = [&]() {
        if (new_pos >= 0) {   // (wave-uniform) the wave whose tiles include the new token's quantises and stores it
            const int nt = new_pos / kTile;
            if (nt >= t && nt < tile_end && (nt - t) % tstep == 0) quantise_new_token<FMT, ROPE>(p, wk, lane, lds_new);
        }
    };
    if constexpr (!ROPE) new_token();
    auto first_tiles = [&]() {
#pragma unroll
        for (int st = 0; st < PF; st++) {
            kspre[st] = vspre[st] = u32x2{0u, 0u};
            if (t + st * tstep < tile_end) {
                fetch(wk.kbase, wk.ksbase, 0, t + st * tstep, kpre[st], kspre[st]);
                fetch(wk.vbase, wk.vsbase, 1, t + st * tstep, vpre[st], vspre[st]);
            }
        }
    };
    // (ROPE: the query's features are rotated as they are loaded, with the sequence's cos / sin rows; four loads per piece
    // instead of one, asked for AHEAD of the first tiles: behind them they would arrive after two tiles of codes)
    const char *cos_row = ROPE ? p.rope_cos + (int64_t)b * p.rope_stride_b : nullptr;
    const char *sin_row = ROPE ? p.rope_sin + (int64_t)b * p.rope_stride_b : nullptr;
    if constexpr (!ROPE) first_tiles();

    // Query operands, one per slice j: in the lanes of group blk_c the 8 features of slice j of block blk_c of head h_c,
    // zeros in the other lane groups.
    //   Q8_0: features 32 blk + 8 j + 0..7
    //   Q4_0: features 32 blk + 4 j + 0..3 (low nibbles) and 32 blk + 16 + 4 j + 0..3 (high nibbles: the codes arrive as
    //         16 u, so these features are divided by 16 -- exact but for subnormal results)
    half8_t qf[NX][NJ];
    float bias[NX];      // minus what the products add up for a block of all-zero-point codes
    const bool mine = qb == blk_c;
    // ROPE: every piece's four loads first, then the first tiles', then the arithmetic (the loads return in order)
    constexpr int NPC = Q8 ? 1 : 2;
    RopeRaw<Q8 ? 8 : 4> raw[ROPE ? NX : 1][ROPE ? NJ : 1][NPC];
    if constexpr (ROPE) {
#pragma unroll
        for (int X = 0; X < NX; X++)
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int sl = qs * NJ + j, f0 = 32 * (X * BPC + blk_c);
                if constexpr (Q8) {
                    raw[X][j][0] = rope_load128<8>(qrow, cos_row, sin_row, f0 + 8 * sl);
                } else {
                    raw[X][j][0] = rope_load128<4>(qrow, cos_row, sin_row, f0 + 4 * sl);
                    raw[X][j][NPC - 1] = rope_load128<4>(qrow, cos_row, sin_row, f0 + 16 + 4 * sl);
                }
            }
        new_token();   // (its own loads join the query's in flight)
        first_tiles();
    }
#pragma unroll
    for (int X = 0; X < NX; X++) {
        float part = 0.0f;
        const _Float16 *qblk = qrow + 32 * (X * BPC + blk_c);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int sl = qs * NJ + j;   // slice of the block
            half8_t f = {0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (Q8) {
                half8_t x;
                if constexpr (ROPE && Q8) x = rope_finish<8>(raw[X][j][0]);
                else x = *reinterpret_cast<const half8_t *>(qblk + 8 * sl);
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) sum += (float)x[i];
                if (mine) f = x, part += 1152.0f * sum;   // the plane holds code + 128, under 1024
            } else {
                half4_t lo, hi;
                if constexpr (ROPE && !Q8) {
                    lo = rope_finish<4>(raw[X][j][0]);
                    hi = rope_finish<4>(raw[X][j][NPC - 1]);
                } else {
                    lo = *reinterpret_cast<const half4_t *>(qblk + 4 * sl);
                    hi = *reinterpret_cast<const half4_t *>(qblk + 16 + 4 * sl);
                }
                half8_t x;
                float s_lo = 0.0f, s_hi = 0.0f, s_hi16 = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const _Float16 h16 = hi[i] * (_Float16)0.0625f;
                    // the order in which nibbles8() delivers the codes of a word: (lo0, lo2), (hi0, hi2), (lo1, lo3), (hi1, hi3)
                    const int at = 4 * (i & 1) + (i >> 1);
                    x[at] = lo[i], x[2 + at] = h16;
                    s_lo += (float)lo[i], s_hi16 += (float)h16, s_hi += 16.0f * (float)h16;
                }
                if (mine) f = x, part += 1024.0f * (s_lo + s_hi16) + 8.0f * (s_lo + s_hi);
            }
            qf[X][j] = f;
        }
        part += __shfl_xor(part, 16, 64);   // the lane groups that hold the column's features hand their sums to the others
        part += __shfl_xor(part, 32, 64);
        bias[X] = -part;
    }
#pragma unroll
    for (int X = 0; X < NX; X++)
#pragma unroll
        for (int j = 0; j < NJ; j++) asm volatile("" : "+v"(qf[X][j]));   // settled here, not at first use inside the loop

    float m_run = -INFINITY, l_run = 0.0f;   // log2 domain, already scaled
    float4_t o16[D / 16];
    float sp[NX];
#pragma unroll
    for (int X = 0; X < NX; X++) sp[X] = 0.0f;
#pragma unroll
    for (int fb = 0; fb < D / 16; fb++) o16[fb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // K fragment of this lane for set X, slice j: token 16 mb + l16 (its key does not depend on mb), block X BPC + qb, the
    // bytes of slice sl = qs NJ + j: Q8_0 chunk 2 block + sl / 2, half sl % 2; Q4_0 chunk block, word sl
    uint32_t k_frag[NX][NJ];
#pragma unroll
    for (int X = 0; X < NX; X++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int blk = X * BPC + qb, sl = qs * NJ + j;
            const int row = RS ? (l16 ^ qb) : l16;   // (RS: the feeders of block blk take the tokens of a group of four in the order t ^ blk)
            k_frag[X][j] = Q8 ? row * RB + 16 * ((2 * blk + (sl >> 1)) ^ key_k(row)) + 8 * (sl & 1) : row * RB + 16 * (blk ^ key_k(row)) + 4 * sl;
        }
    // V^T fragments: as in the block-scaling body
    // (RS: position 2 j + mb of the contraction is token 16 mb + 4 q4 + j; Q4_0's nibbles8() delivers byte p of the eight at
    // position (0, 2, 1, 3, 4, 6, 5, 7)[p])
    const int vk = l16 >> 1;
    const int v_tok = !RS ? (vk < 4 ? 4 * q4 + vk : 12 + 4 * q4 + vk)
                          : Q8 ? 16 * (vk & 1) + 4 * q4 + (vk >> 1) : 16 * ((vk >> 1) & 1) + 4 * q4 + 2 * (vk >> 2) + (vk & 1);
    const unsigned char *v_row = lds_v + v_tok * RB + 8 * (l16 & 1);
    const uint32_t v_key16 = 16 * key_v(v_tok);
    // block scales of this lane's tokens 16 mb + 4 q4 + 0..3 in its block blk_c of set 0 (set X: X BPC block rows on): 8
    // contiguous bytes per mb
    // (RS: the V scales of a lane's eight tokens are 16 contiguous bytes, pairs (token j of the first half, of the second))
    const unsigned char *ks_frag = lds_ks + (blk_c * kTile + 4 * q4) * 2, *vs_frag = lds_vs + (blk_c * kTile + (RS ? 8 : 4) * q4) * 2;
    // where token `lane` goes in a row of the scale tiles: Q4_0 pairs tokens (0, 2) and (1, 3) of a group of four, the
    // order in which nibbles8() delivers the V codes (and so the order of the probabilities in their operand)
    const int sc_pos = Q8 ? lane : ((lane & ~3) | ((lane & 1) << 1) | ((lane >> 1) & 1));
    // RS: in block row blk of the K scales token t sits at t ^ (blk % BPC), the order of the score registers; in
    // every block row of the V scales token 16 mb + 4 q + j sits at 8 q + 2 j + mb
    const int vs_pos = 8 * ((lane & 15) >> 2) + 2 * (lane & 3) + ((lane >> 4) & 1);
    const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
    const NibbleConsts nc = nibble_consts();
    auto ror_add = [](float x, auto ctrl_tag) {   // x + (x of the lane `n` places on in its row of 16 lanes)
        constexpr int ctrl = decltype(ctrl_tag)::value;
        const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, 0xf, false);
        return x + __builtin_bit_cast(float, y);
    };

    const float c_log2 = p.scale_log2;   // > 0 (checked on the host): the maximum is taken before scaling
    auto do_tile = [&](auto stage_tag, int t) {
        constexpr int ST = decltype(stage_tag)::value;
        const int t0 = t * kTile;
        const bool more = t + PF * tstep < tile_end;
        // ---- this tile's codes and scales -> LDS, the tile PF steps on into flight --------------------------------
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            *reinterpret_cast<u32x4 *>(lds_k + k_slot[j]) = kpre[ST][j];
            *reinterpret_cast<u32x4 *>(lds_v + v_slot[j]) = vpre[ST][j];
        }
        if (lane < kTile) {   // token `lane`: its four block scales to the four block rows of the transposed tiles
            uint16_t *ksT = reinterpret_cast<uint16_t *>(lds_ks) + (RS ? 0 : sc_pos), *vsT = reinterpret_cast<uint16_t *>(lds_vs) + (RS ? vs_pos : sc_pos);
            if constexpr (RS) {
                ksT[lane] = (uint16_t)kspre[ST].x, ksT[kTile + (lane ^ (1 % BPC))] = (uint16_t)(kspre[ST].x >> 16);
                ksT[2 * kTile + (lane ^ (2 % BPC))] = (uint16_t)kspre[ST].y, ksT[3 * kTile + (lane ^ (3 % BPC))] = (uint16_t)(kspre[ST].y >> 16);
            } else {
                ksT[0] = (uint16_t)kspre[ST].x, ksT[kTile] = (uint16_t)(kspre[ST].x >> 16);
                ksT[2 * kTile] = (uint16_t)kspre[ST].y, ksT[3 * kTile] = (uint16_t)(kspre[ST].y >> 16);
            }
            vsT[0] = (uint16_t)vspre[ST].x, vsT[kTile] = (uint16_t)(vspre[ST].x >> 16);
            vsT[2 * kTile] = (uint16_t)vspre[ST].y, vsT[3 * kTile] = (uint16_t)(vspre[ST].y >> 16);
        }
        if (more) {
            fetch(wk.kbase, wk.ksbase, 0, t + PF * tstep, kpre[ST], kspre[ST]);
            fetch(wk.vbase, wk.vsbase, 1, t + PF * tstep, vpre[ST], vspre[ST]);
        }
        // ---- codes x block-diagonal query operands: column (blk, h) receives the sum over block X BPC + blk ----------------
        float4_t acc[NX][2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
#pragma unroll
            for (int X = 0; X < NX; X++) {
                acc[X][mb] = float4_t{bias[X], bias[X], bias[X], bias[X]};
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    half8_t kf;
                    if constexpr (Q8) {
                        const u32x2 c = *reinterpret_cast<const u32x2 *>(lds_k + k_frag[X][j] + 16 * mb * RB);
                        kf = magic8(c.x, c.y);   // (the plane holds code + 128)
                    } else {
                        const uint32_t c = *reinterpret_cast<const uint32_t *>(lds_k + k_frag[X][j] + 16 * mb * RB);
                        uint32_t r0, r1, r2, r3;
                        nibbles8(nc, c, r0, r1, r2, r3);
                        kf = __builtin_bit_cast(half8_t, u32x4{r0, r1, r2, r3});
                    }
                    acc[X][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[X][j], acc[X][mb], 0, 0, 0);
                }
            }
        }
        half2_t pf[4];
        if constexpr (RS) {
            // ---- this block's share of the scores of tokens 16 mb + 4 q4 + (r ^ blk_c), then the reduce-scatter over the quad ---
            auto quad_add = [](float x, float y, auto ctrl_tag) {   // x + (y of the lane across in the quad)
                constexpr int ctrl = decltype(ctrl_tag)::value;
                const int o = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, y), ctrl, 0xf, 0xf, false);
                return x + __builtin_bit_cast(float, o);
            };
            // Maxima as the bare instruction: fmaxf first copies every operand that might be a signalling NaN through a
            // canonicalising v_max (nine more instructions per tile here).  The quad steps read their operand through DPP;
            // the two wait states such a read needs after the write of its register are in the asm, because the compiler
            // does not count wait states for registers that an asm writes.
            auto vmax = [](float a, float b) {
                float r;
                asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
                return r;
            };
            auto quad_max_swap1 = [](float x) {
                float r;
                asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(r) : "v"(x));
                return r;
            };
            auto quad_max_swap2 = [](float x) {
                float r;
                asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(r) : "v"(x));
                return r;
            };
            using Swap1 = std::integral_constant<int, 0xB1>;   // quad_perm:[1,0,3,2]
            using Swap2 = std::integral_constant<int, 0x4E>;   // quad_perm:[2,3,0,1]
            constexpr int NS = 4 / BPC;   // scores per lane and half: tokens blk_c + BPC i
            float x[2][4];
#pragma unroll
            for (int mb = 0; mb < 2; mb++) {
#pragma unroll
                for (int X = 0; X < NX; X++) {
                    const u32x2 dk = *reinterpret_cast<const u32x2 *>(ks_frag + X * BPC * kTile * 2 + 32 * mb);
                    const half2_t da = as_half2(dk.x), db = as_half2(dk.y);
                    const _Float16 dv[4] = {da[0], da[1], db[0], db[1]};
#pragma unroll
                    for (int r = 0; r < 4; r++) x[mb][r] = __builtin_fmaf((float)dv[r], acc[X][mb][r], X == 0 ? 0.0f : x[mb][r]);
                }
            }
            float z[2][NS];
            {
                float y[2], wv[2];
#pragma unroll
                for (int mb = 0; mb < 2; mb++) y[mb] = quad_add(x[mb][0], x[mb][1], Swap1{}), wv[mb] = quad_add(x[mb][2], x[mb][3], Swap1{});
#pragma unroll
                for (int mb = 0; mb < 2; mb++) {
                    if constexpr (H == 4) z[mb][0] = quad_add(y[mb], wv[mb], Swap2{});   // token 16 mb + 4 q4 + blk_c, head h_c
                    else z[mb][0] = y[mb], z[mb][NS - 1] = wv[mb];                       // tokens 16 mb + 4 q4 + blk_c (+ 2)
                }
            }
            if (t0 + kTile > T) {   // the sequence's last tile: tokens past its end do not count
                asm volatile("");   // (a branch, not selects in every tile)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int i = 0; i < NS; i++)
                        if (t0 + 16 * mb + 4 * q4 + blk_c + BPC * i >= T) z[mb][i] = -INFINITY;
            }
            float tmax = vmax(z[0][0], z[1][0]);
            if constexpr (NS == 2) tmax = vmax(tmax, vmax(z[0][NS - 1], z[1][NS - 1]));
            tmax = quad_max_swap1(tmax);
            if constexpr (H == 4) tmax = quad_max_swap2(tmax);
            tmax = vmax(tmax, __shfl_xor(tmax, 16, 64));
            tmax = vmax(tmax, __shfl_xor(tmax, 32, 64));
            const float m_new = vmax(m_run, tmax * c_log2);   // finite: every tile holds at least one valid token
            float psum = 0.0f;
            uint32_t mine2[NS];
#pragma unroll
            for (int i = 0; i < NS; i++) {
                const float p0 = fast_exp2(__builtin_fmaf(z[0][i], c_log2, -m_new)), p1 = fast_exp2(__builtin_fmaf(z[1][i], c_log2, -m_new));
                psum += p0 + p1;
                mine2[i] = __builtin_bit_cast(uint32_t, half2_t{(_Float16)p0, (_Float16)p1});
            }
            // register j of every lane: the pair of token j of the lane's group of four (quad broadcasts from the lane that
            // holds it: lane j of the quad; with two lanes per head lane j % 2 of the head's pair, its register j / 2)
            if constexpr (H == 4) {
                pf[0] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0x00, 0xf, 0xf, true));
                pf[1] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0x55, 0xf, 0xf, true));
                pf[2] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0xAA, 0xf, 0xf, true));
                pf[3] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0xFF, 0xf, 0xf, true));
            } else {
                pf[0] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0xA0, 0xf, 0xf, true));        // quad_perm:[0,0,2,2]
                pf[1] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[0], 0xF5, 0xf, 0xf, true));        // quad_perm:[1,1,3,3]
                pf[2] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[NS - 1], 0xA0, 0xf, 0xf, true));
                pf[3] = as_half2((uint32_t)__builtin_amdgcn_mov_dpp((int)mine2[NS - 1], 0xF5, 0xf, 0xf, true));
            }
            const bool moved = m_new != m_run;
            const float alpha = fast_exp2(m_run - m_new);
            l_run = l_run * alpha + psum;   // this lane's own tokens; the lanes of a head are added up after the loop
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
                for (int fb = 0; fb < D / 16; fb++) o16[fb] *= alpha;
#pragma unroll
                for (int X = 0; X < NX; X++) sp[X] *= alpha;
            }
        } else {
        // ---- scores (before the softmax scale) of tokens 16 mb + 4 q4 + r for head h_c: this lane's blocks, then all four --
        float sc8[8];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
#pragma unroll
            for (int X = 0; X < NX; X++) {
                const u32x2 dk = *reinterpret_cast<const u32x2 *>(ks_frag + X * BPC * kTile * 2 + 32 * mb);   // scales of tokens r = 0, 1 | 2, 3
                const half2_t da = as_half2(dk.x), db = as_half2(dk.y);
                // (Q4_0: the scale tiles hold a group of four tokens in the order 0, 2, 1, 3)
                const _Float16 dv[4] = {da[0], Q8 ? da[1] : db[0], Q8 ? db[0] : da[1], db[1]};
#pragma unroll
                for (int r = 0; r < 4; r++) sc8[4 * mb + r] = __builtin_fmaf((float)dv[r], acc[X][mb][r], X == 0 ? 0.0f : sc8[4 * mb + r]);
            }
        }
        // the blocks of a head sit H lanes apart in a row of 16 lanes: rotations add them up in every lane.  (One stage at a
        // time over all eight values: a rotation must wait two issue slots for its operand, and a value carried through
        // both stages on its own fills them with s_nop.)
        if constexpr (H == 4) {
#pragma unroll
            for (int i = 0; i < 8; i++) sc8[i] = ror_add(sc8[i], std::integral_constant<int, 0x124>{});   // row_ror:4
        }
#pragma unroll
        for (int i = 0; i < 8; i++) sc8[i] = ror_add(sc8[i], std::integral_constant<int, 0x128>{});   // row_ror:8

        if (t0 + kTile > T) {   // the sequence's last tile: tokens past its end do not count
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (t0 + 16 * (i >> 2) + 4 * q4 + (i & 3) >= T) sc8[i] = -INFINITY;
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; i++) tmax = fmaxf(tmax, sc8[i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax * c_log2);   // finite: every tile holds at least one valid token
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // Q8_0: tokens (2i, 2i + 1) of the lane's eight; Q4_0: (0, 2), (1, 3), (4, 6), (5, 7)
            const int ia = Q8 ? 2 * i : 4 * (i >> 1) + (i & 1), ib = Q8 ? 2 * i + 1 : ia + 2;
            const float p0 = fast_exp2(__builtin_fmaf(sc8[ia], c_log2, -m_new)), p1 = fast_exp2(__builtin_fmaf(sc8[ib], c_log2, -m_new));
            psum += p0 + p1;
            pf[i] = half2_t{(_Float16)p0, (_Float16)p1};
        }
        const bool moved = m_new != m_run;
        const float alpha = fast_exp2(m_run - m_new);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int fb = 0; fb < D / 16; fb++) o16[fb] *= alpha;
#pragma unroll
            for (int X = 0; X < NX; X++) sp[X] *= alpha;
        }
        }
        // ---- probabilities times the V scales of their tokens in block X BPC + blk_c: one operand per set of blocks ---------
        // pf[i] holds two tokens of 4 q4 + 0..3 for i < 2 and of 16 + 4 q4 + 0..3 for i >= 2, the scale tiles the same pairs
        half8_t pb[NX];
#pragma unroll
        for (int X = 0; X < NX; X++) {
            const unsigned char *vsx = vs_frag + X * BPC * kTile * 2;
            uint32_t ev[4];
            if constexpr (RS) {
                const u32x4 e = *reinterpret_cast<const u32x4 *>(vsx);
                ev[0] = e.x, ev[1] = e.y, ev[2] = e.z, ev[3] = e.w;
            } else {
                const u32x2 e0 = *reinterpret_cast<const u32x2 *>(vsx), e1 = *reinterpret_cast<const u32x2 *>(vsx + 32);
                ev[0] = e0.x, ev[1] = e0.y, ev[2] = e1.x, ev[3] = e1.y;
            }
            u32x4 pw;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t pp = pf[i] * as_half2(ev[i]);
                sp[X] = __builtin_amdgcn_fdot2(pp, ones, sp[X], false);
                pw[i] = __builtin_bit_cast(uint32_t, pp);
            }
            pb[X] = __builtin_bit_cast(half8_t, pw);
        }
        // ---- O^T += codes^T x scaled probabilities: the tile of block blk is right in the columns (blk % BPC, h) -------------
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            if constexpr (Q8) {
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    uint32_t w0, w1;
                    lds_read_tr8(v_row + ((32 * blk + 16 * hf) ^ v_key16), w0, w1);
                    const half8_t vf = magic8(w0, w1);
                    o16[2 * blk + hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pb[blk / BPC], o16[2 * blk + hf], 0, 0, 0);
                }
            } else {
                uint32_t w0, w1;   // byte l16 of the block's 16: feature l16 in the low nibble, 16 + l16 in the high one
                lds_read_tr8(v_row + ((16 * blk) ^ v_key16), w0, w1);
                uint32_t la, ha, lb, hb2, lc, hc, ld2, hd;   // tokens (0, 2), (1, 3) of w0's four, then of w1's
                nibbles8(nc, w0, la, ha, lb, hb2);
                nibbles8(nc, w1, lc, hc, ld2, hd);
                const half8_t vlo = __builtin_bit_cast(half8_t, u32x4{la, lb, lc, ld2}), vhi = __builtin_bit_cast(half8_t, u32x4{ha, hb2, hc, hd});
                o16[2 * blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vlo, pb[blk / BPC], o16[2 * blk], 0, 0, 0);
                o16[2 * blk + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vhi, pb[blk / BPC], o16[2 * blk + 1], 0, 0, 0);
            }
        }
    };
    static_assert(PF <= 2, "stages are written out");
    while (t < tile_end) {
        do_tile(std::integral_constant<int, 0>{}, t);
        t += tstep;
        if constexpr (PF > 1) {
            if (t < tile_end) do_tile(std::integral_constant<int, 1>{}, t), t += tstep;
        }
    }
    if constexpr (RS) {   // a lane has summed its own tokens of every tile
        l_run += __shfl_xor(l_run, 1, 64);
        if constexpr (H == 4) l_run += __shfl_xor(l_run, 2, 64);
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    // the zero points of this lane's column: O[f, h] -= (1024 + zero) * SP[h, blk] (Q4_0's high features arrived 16 times
    // too large); only the tiles of the blocks X BPC + blk_c are read off this column
#pragma unroll
    for (int X = 0; X < NX; X++) {
        sp[X] += __shfl_xor(sp[X], 16, 64);
        sp[X] += __shfl_xor(sp[X], 32, 64);
    }
#pragma unroll
    for (int blk = 0; blk < NB; blk++) {
        const float spb = sp[blk / BPC];
        if constexpr (Q8) {
            o16[2 * blk] -= 1152.0f * spb;
            o16[2 * blk + 1] -= 1152.0f * spb;
        } else {
            o16[2 * blk] -= 1032.0f * spb;
            o16[2 * blk + 1] = o16[2 * blk + 1] * 0.0625f - 72.0f * spb;
        }
    }

    // ---- merge the 4 waves through LDS (the tiles are dead): rows 0..H-1 are the heads, with H = 4 rows 4..7 neutral records -
    __syncthreads();
    float *comb = reinterpret_cast<float *>(lds_raw);   // [kWaves][GP*D + 2*GP]
    {
        float *cw = comb + w * kCombStride;
        const float4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int fb = 0; fb < D / 16; fb++)
            if ((fb >> 1) % BPC == blk_c) {
                *reinterpret_cast<float4_t *>(cw + h_c * D + 16 * fb + 4 * q4) = o16[fb];
                if constexpr (H == 4) *reinterpret_cast<float4_t *>(cw + (4 + h_c) * D + 16 * fb + 4 * q4) = zero4;
            }
        if (q4 == 0 && blk_c == 0) {
            cw[GP * D + h_c] = m_run;
            cw[GP * D + GP + h_c] = l_run;
            if constexpr (H == 4) {
                cw[GP * D + 4 + h_c] = -INFINITY;
                cw[GP * D + GP + 4 + h_c] = 0.0f;
            }
        }
    }
    wave_records_to_output<D, GP>(p, wk, lds_raw, head0, g, tid);
}

// Affine u8 caches as QuantizedKvSdpa keeps them (kv_quant.rs:105-236): K[t, c] = lo_k[c] + u_k[t, c] * s_k[c] with one
// (lo, scale) per channel for the whole sequence, V[t, f] = lo_v[t] + u_v[t, f] * s_v[t] per token.  Nothing is
// dequantised:
//   S[t, h] = sum_c (q[h, c] s_k[c]) u_k[t, c]  +  sum_c q[h, c] lo_k[c]
// and the second term is the same for every token of a head, so the softmax does not see it: the query features are
// scaled once per launch and the raw codes go into the matrix cores as the exact halves 1024 + u (the 1024 leaves through
// the accumulator's initial value);
//   O[h, f] = sum_t (P[t, h] s_v[t]) u_v[t, f]  +  sum_t P[t, h] lo_v[t]
// with the token scales folded into the probabilities (one operand for the whole row) and the second term one scalar per
// head, added to every feature after the loop.  Lane layout, LDS tiles and the combine are those of the block-scaling
// body; wk.ksbase / wk.vsbase are the Values' per-token scale and lo rows (f32).
template <int GP, int PF>
__device__ __forceinline__ void decode_mfma_kivi_body(const DecodeDev &p, const MfmaWork &wk) {
    static_assert(GP <= 16, "the 16-wide layout: at most 16 heads");
    constexpr int D = 128;
    constexpr int NB = D / 32;
    constexpr int RB = D;                      // code bytes per token row
    constexpr int NLD = kTile * RB / 1024;     // 128-bit loads per lane, tile and tensor
    constexpr int CPR = RB / 16;
    constexpr int kCodeBytes = kTile * RB;
    constexpr int kParamBytes = 2 * kTile * 4; // the tile's token scales, then its token los
    constexpr int kWaveBytes = 2 * kCodeBytes + kParamBytes;
    constexpr int kCombStride = GP * D + 2 * GP;
    constexpr int kLdsBytes = kWaves * (kWaveBytes > kCombStride * 4 ? kWaveBytes : kCombStride * 4);
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLdsBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, q4 = lane >> 4;
    const int kvh = wk.kvh, b = wk.seq;
    const int g = p.g_real;
    unsigned char *lds_k = lds_raw + w * kWaveBytes, *lds_v = lds_k + kCodeBytes;
    float *lds_vp = reinterpret_cast<float *>(lds_v + kCodeBytes);

    const int64_t head0 = (int64_t)b * p.Hq + (int64_t)kvh * g;
    const _Float16 *qrow = reinterpret_cast<const _Float16 *>(p.q) + (head0 + min(l16, g - 1)) * D;
    const float *ksc = p.chan_scale + ((int64_t)b * p.Hkv + kvh) * D;
    const int T = wk.T;
    const int tile_begin = wk.tile_begin, tile_end = wk.tile_end;
    // lanes 0..31 carry the scale of token `lane` of a tile, lanes 32..63 the lo of token `lane - 32`
    const float *par_row = reinterpret_cast<const float *>(lane < kTile ? wk.ksbase : wk.vsbase);

    u32x4 kpre[PF][NLD], vpre[PF][NLD];
    float ppre[PF];
    auto fetch = [&](int t, u32x4 (&kd)[NLD], u32x4 (&vd)[NLD], float &par) {
        const int t0 = t * kTile;
        const char *kb = wk.kbase + (int64_t)t0 * RB, *vb = wk.vbase + (int64_t)t0 * RB;
        if (t0 + kTile <= T) {
#pragma unroll
            for (int j = 0; j < NLD; j++) {
                kd[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(kb + (j * 64 + lane) * 16));
                vd[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(vb + (j * 64 + lane) * 16));
            }
            par = par_row[t0 + (lane & (kTile - 1))];
        } else {   // rows past the end of the sequence repeat its last token (their scores are masked below)
            const int last = T - 1 - t0;
#pragma unroll
            for (int j = 0; j < NLD; j++) {
                const int c = j * 64 + lane, row = min(c / CPR, last), dc = c % CPR;
                kd[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(kb + row * RB + dc * 16));
                vd[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(vb + row * RB + dc * 16));
            }
            par = par_row[t0 + min(lane & (kTile - 1), last)];
        }
    };
    auto key_k = [](int row) { return row & 7; };
    auto key_v = [](int row) { return (row & 3) | (((row >> 4) & 1) << 2); };
    uint32_t k_slot[NLD], v_slot[NLD];
#pragma unroll
    for (int j = 0; j < NLD; j++) {
        const int c = j * 64 + lane, row = c / CPR, dc = c % CPR;
        k_slot[j] = row * RB + 16 * (dc ^ key_k(row));
        v_slot[j] = row * RB + 16 * (dc ^ key_v(row));
    }
    const int tstep = wk.tile_step;
    int t = tile_begin + w;
#pragma unroll
    for (int st = 0; st < PF; st++) {
        ppre[st] = 0.0f;
        if (t + st * tstep < tile_end) fetch(t + st * tstep, kpre[st], vpre[st], ppre[st]);
    }

    // Q^T fragments of this lane's head, one per 32 channels: channels 32 blk + 8 q4 + 0..7, times their key scales
    // The products q * s_k go to the matrix cores as halves: a power of two takes the largest key scale of this kv head
    // into [1/2, 1) first and leaves through the score scale below, so that keys of any magnitude keep the halves'
    // 11 bits (scales under 6e-5 would otherwise make every product a subnormal half).
    half8_t qf[NB];
    float ks_max = 0.0f;
    float4_t ksv[NB][2];
#pragma unroll
    for (int blk = 0; blk < NB; blk++) {
        ksv[blk][0] = *reinterpret_cast<const float4_t *>(ksc + 32 * blk + 8 * q4);
        ksv[blk][1] = *reinterpret_cast<const float4_t *>(ksc + 32 * blk + 8 * q4 + 4);
#pragma unroll
        for (int i = 0; i < 8; i++) ks_max = fmaxf(ks_max, fabsf(ksv[blk][i >> 2][i & 3]));
    }
    ks_max = fmaxf(ks_max, __shfl_xor(ks_max, 16, 64));
    ks_max = fmaxf(ks_max, __shfl_xor(ks_max, 32, 64));
    const float k_norm = pow2_normaliser(ks_max), k_denorm = 1.0f / k_norm;   // exact powers of two
    float part = 0.0f;
#pragma unroll
    for (int blk = 0; blk < NB; blk++) {
        const half8_t x = *reinterpret_cast<const half8_t *>(qrow + 32 * blk + 8 * q4);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            qf[blk][i] = (_Float16)((float)x[i] * (ksv[blk][i >> 2][i & 3] * k_norm));
            part += (float)qf[blk][i];
        }
    }
    part += __shfl_xor(part, 16, 64);
    part += __shfl_xor(part, 32, 64);
    const float bias = -1024.0f * part;
#pragma unroll
    for (int blk = 0; blk < NB; blk++) asm volatile("" : "+v"(qf[blk]));   // settled here, not at first use inside the loop

    float m_run = -INFINITY, l_run = 0.0f;   // log2 domain, already scaled
    float4_t o16[D / 16];
    float sp = 0.0f, sl = 0.0f;              // sum of P s_v (as the halves the matrix cores saw), sum of P lo_v
#pragma unroll
    for (int fb = 0; fb < D / 16; fb++) o16[fb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    uint32_t k_frag[NB];
#pragma unroll
    for (int blk = 0; blk < NB; blk++) k_frag[blk] = l16 * RB + 16 * ((2 * blk + (q4 >> 1)) ^ key_k(l16)) + 8 * (q4 & 1);
    const int vk = l16 >> 1, v_tok = vk < 4 ? 4 * q4 + vk : 12 + 4 * q4 + vk;
    const unsigned char *v_row = lds_v + v_tok * RB + 8 * (l16 & 1);
    const uint32_t v_key16 = 16 * key_v(v_tok);
    const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};

    const float c_log2 = p.scale_log2 * k_denorm;   // > 0 (checked on the host): the maximum is taken before scaling
    // Likewise P * s_v: v_norm is the power of two that takes the largest Value scale seen so far into [1/2, 1); when a
    // tile brings a larger one the accumulated products move to the new factor (exact), like the running maximum.
    float v_norm = 0.0f;   // 0: no tile yet
    auto do_tile = [&](auto stage_tag, int t) {
        constexpr int ST = decltype(stage_tag)::value;
        const int t0 = t * kTile;
        const bool more = t + PF * tstep < tile_end;
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            *reinterpret_cast<u32x4 *>(lds_k + k_slot[j]) = kpre[ST][j];
            *reinterpret_cast<u32x4 *>(lds_v + v_slot[j]) = vpre[ST][j];
        }
        lds_vp[lane] = ppre[ST];
        if (more) fetch(t + PF * tstep, kpre[ST], vpre[ST], ppre[ST]);
        // ---- codes x scaled query features, all 128 channels into one accumulator ------------------------------------
        float sc8[8];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
            float4_t acc = {bias, bias, bias, bias};
#pragma unroll
            for (int blk = 0; blk < NB; blk++) {
                const u32x2 c = *reinterpret_cast<const u32x2 *>(lds_k + k_frag[blk] + 16 * mb * RB);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(magic8(c.x, c.y), qf[blk], acc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) sc8[4 * mb + r] = acc[r];   // tokens 16 mb + 4 q4 + r, head l16
        }
        if (t0 + kTile > T) {   // the sequence's last tile: tokens past its end do not count
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (t0 + 16 * (i >> 2) + 4 * q4 + (i & 3) >= T) sc8[i] = -INFINITY;
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; i++) tmax = fmaxf(tmax, sc8[i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax * c_log2);   // finite: every tile holds at least one valid token
        float pe[8], psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            pe[i] = fast_exp2(__builtin_fmaf(sc8[i], c_log2, -m_new));
            psum += pe[i];
        }
        const bool moved = m_new != m_run;
        const float alpha = fast_exp2(m_run - m_new);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int fb = 0; fb < D / 16; fb++) o16[fb] *= alpha;
            sp *= alpha;
            sl *= alpha;
        }
        // ---- probabilities times the scales of their tokens: one operand for the whole row ---------------------------------
        u32x4 pw;
        {
            const float4_t sa = *reinterpret_cast<const float4_t *>(lds_vp + 4 * q4), sb = *reinterpret_cast<const float4_t *>(lds_vp + 16 + 4 * q4);
            const float4_t la = *reinterpret_cast<const float4_t *>(lds_vp + kTile + 4 * q4), lb = *reinterpret_cast<const float4_t *>(lds_vp + kTile + 16 + 4 * q4);
            const float sv[8] = {sa[0], sa[1], sa[2], sa[3], sb[0], sb[1], sb[2], sb[3]};
            const float lv[8] = {la[0], la[1], la[2], la[3], lb[0], lb[1], lb[2], lb[3]};
            float sv_max = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) sv_max = fmaxf(sv_max, fabsf(sv[i]));
            sv_max = fmaxf(sv_max, __shfl_xor(sv_max, 16, 64));
            sv_max = fmaxf(sv_max, __shfl_xor(sv_max, 32, 64));   // the tile's 32 tokens: the same value in every lane
            const float want = pow2_normaliser(sv_max);
            if (v_norm == 0.0f) {
                v_norm = want;
            } else if (want < v_norm) {   // a larger scale than any before (wave-uniform)
                const float f = want / v_norm;   // a power of two below 1
#pragma unroll
                for (int fb = 0; fb < D / 16; fb++) o16[fb] *= f;
                sp *= f;
                v_norm = want;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t pp = {(_Float16)(pe[2 * i] * (sv[2 * i] * v_norm)), (_Float16)(pe[2 * i + 1] * (sv[2 * i + 1] * v_norm))};
                sp = __builtin_amdgcn_fdot2(pp, ones, sp, false);
                sl = __builtin_fmaf(pe[2 * i], lv[2 * i], sl);
                sl = __builtin_fmaf(pe[2 * i + 1], lv[2 * i + 1], sl);
                pw[i] = __builtin_bit_cast(uint32_t, pp);
            }
        }
        const half8_t pb = __builtin_bit_cast(half8_t, pw);
        // ---- O^T += codes^T x scaled probabilities -----------------------------------------------------------------------
#pragma unroll
        for (int fb = 0; fb < D / 16; fb++) {
            uint32_t w0, w1;
            lds_read_tr8(v_row + ((16 * fb) ^ v_key16), w0, w1);
            o16[fb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(magic8(w0, w1), pb, o16[fb], 0, 0, 0);
        }
    };
    static_assert(PF <= 2, "stages are written out");
    while (t < tile_end) {
        do_tile(std::integral_constant<int, 0>{}, t);
        t += tstep;
        if constexpr (PF > 1) {
            if (t < tile_end) do_tile(std::integral_constant<int, 1>{}, t), t += tstep;
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    sp += __shfl_xor(sp, 16, 64);
    sp += __shfl_xor(sp, 32, 64);
    sl += __shfl_xor(sl, 16, 64);
    sl += __shfl_xor(sl, 32, 64);
    // the 1024 under every code leaves, the power of two of the Value scales leaves, the tokens' los arrive
    const float v_denorm = v_norm > 0.0f ? 1.0f / v_norm : 0.0f;
    const float shift = 1024.0f * sp;
#pragma unroll
    for (int fb = 0; fb < D / 16; fb++)
#pragma unroll
        for (int r = 0; r < 4; r++) o16[fb][r] = __builtin_fmaf(o16[fb][r] - shift, v_denorm, sl);

    // ---- merge the 4 waves through LDS (the tiles are dead) ------------------------------------------------------------
    __syncthreads();
    float *comb = reinterpret_cast<float *>(lds_raw);   // [kWaves][GP*D + 2*GP]
    if (l16 < GP) {
        float *cw = comb + w * kCombStride;
#pragma unroll
        for (int fb = 0; fb < D / 16; fb++) *reinterpret_cast<float4_t *>(cw + l16 * D + 16 * fb + 4 * q4) = o16[fb];
        if (q4 == 0) {
            cw[GP * D + l16] = m_run;
            cw[GP * D + GP + l16] = l_run;
        }
    }
    wave_records_to_output<D, GP>(p, wk, lds_raw, head0, g, tid);
}

// The reference states a ragged batch as a dense batch padded to the longest sequence, with a mask row per
// sequence whose padded columns hold the format's minimum or -inf (flash_sdpa.rs:261-268).  The tokens of such a
// suffix weigh exactly nothing (their exponentials underflow to zero next to any token that counts), so the
// workgroups of a sequence find where it starts and divide only the tokens before it among themselves.
// Returns the number of leading columns to keep: one past the last column of `row` above -60000, or T when no
// column is (a row masked out entirely keeps its tokens: they then weigh the same, as in the reference).
// All threads of the workgroup call it; `red` is kWaves ints of LDS.
__device__ __forceinline__ int mask_row_len(const _Float16 *__restrict__ row, int T, int tid, int *red) {
    int best = -1;   // (T % 4 == 0 and 8-byte aligned rows: checked on the host)
#pragma unroll 8
    for (int c = tid * 4; c < T; c += kThreads * 4) {
        const half4_t v = *reinterpret_cast<const half4_t *>(row + c);
        const _Float16 big = fmaxf(fmaxf((float)v[0], (float)v[1]), fmaxf((float)v[2], (float)v[3]));
        if (big > (_Float16)-60000.0f) {   // the highest column of these four that counts
            const int i = v[3] > (_Float16)-60000.0f ? 3 : v[2] > (_Float16)-60000.0f ? 2 : v[1] > (_Float16)-60000.0f ? 1 : 0;
            best = c + i;   // columns grow with the loop: the last one found is the highest
        }
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) best = max(best, __shfl_xor(best, d, 64));
    if ((tid & 63) == 0) red[tid >> 6] = best;
    __syncthreads();
#pragma unroll
    for (int ww = 0; ww < kWaves; ww++) best = max(best, red[ww]);
    return best < 0 ? T : best + 1;
}

// Dense batch: grid (splits, kv_heads, batch); every sequence has the same length.
// QB: quantised caches on the 16-wide tiles run the body that scales per block outside the products.
template <int D, int GP, int FMT, bool MASK = false, bool W16 = false, int QB = 0>
__global__ __launch_bounds__(kThreads, (QB ? QB % 10 : 2)) void sdpa_decode_mfma_kernel(DecodeDev p) {   // QB = 100 * (1: diagonal, 2: affine u8, 3: diagonal with 8 heads across the columns, 4 / 5: 1 / 3 with the reduce-scatter, 6 / 7: 4 / 5 rotating q and k_new (RoPE), 9: the f16 body doing so) + 10 * tiles ahead + workgroups per CU
    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    MfmaWork wk;
    wk.seq = b, wk.kvh = kvh;
    wk.kbase = p.k + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    wk.vbase = p.v + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    wk.ksbase = wk.vsbase = nullptr;
    if constexpr (FMT != TROCM_F16) {
        wk.ksbase = p.k_scales + (int64_t)b * p.sc_stride_b + (int64_t)kvh * p.sc_stride_h;
        wk.vsbase = p.v_scales + (int64_t)b * p.sc_stride_b + (int64_t)kvh * p.sc_stride_h;
    }
    wk.T = p.T;
    int tiles_per_split = p.tiles_per_split;
    if constexpr (MASK && (W16 || D == 64)) {   // (the 32-wide instantiation at head_dim 128 has no register left for it)
        if (p.mask_stride_h == 0) {   // one mask row for all heads of the sequence: a padded suffix is skipped
            __shared__ int red[kWaves];
            wk.T = mask_row_len(reinterpret_cast<const _Float16 *>(p.mask + (int64_t)b * p.mask_stride_b), p.T, threadIdx.x, red);
            tiles_per_split = ((wk.T + kTile - 1) / kTile + p.nsplit - 1) / p.nsplit;
        }
    }
    const int n_tiles = (wk.T + kTile - 1) / kTile;
    wk.skew_period = 0, wk.skew_split = split;
    if (p.interleave) {   // concurrent workgroups read neighbouring addresses
        wk.tile_begin = split * kWaves, wk.tile_end = n_tiles, wk.tile_step = kWaves * p.nsplit;
        if constexpr (QB == 0 || QB / 100 == 9)
            if (p.xcd_skew >= 2 && p.nsplit % 2 == 0) wk.skew_period = p.xcd_skew;
    } else {
        wk.tile_begin = split * tiles_per_split;
        wk.tile_end = min(n_tiles, wk.tile_begin + tiles_per_split);
        wk.tile_step = kWaves;
    }
    wk.nsplit = p.nsplit;
    const int64_t bh = (int64_t)b * p.Hkv + kvh;
    wk.slot = bh * p.nsplit + split;
    wk.new_pos = p.k_new ? p.new_pos : -1;
    wk.counter = p.counters ? p.counters + bh : nullptr;
    wk.part_first = bh * p.nsplit, wk.part_stride = 1;
    wk.mask = MASK ? p.mask + (int64_t)b * p.mask_stride_b + (int64_t)kvh * p.g_real * p.mask_stride_h : nullptr;
    if constexpr (QB / 100 == 9)
        decode_mfma_body<D, GP, FMT, MASK, W16, true>(p, wk);
    else if constexpr (QB / 100 == 2)
        decode_mfma_kivi_body<GP, (QB / 10) % 10>(p, wk);
    else if constexpr (QB >= 100)
        decode_mfma_qdiag_body<GP, FMT, (QB / 10) % 10, (QB / 100 == 3 || QB / 100 == 5 || QB / 100 == 7 ? 8 : 4), (QB / 100 >= 4), (QB / 100 >= 6)>(p, wk);
    else if constexpr (QB != 0)
        decode_mfma_qblock_body<GP, FMT, QB / 10>(p, wk);
    else
        decode_mfma_body<D, GP, FMT, MASK, W16>(p, wk);
}

// Ragged batch: grid (work items, kv_heads); an item is a tile range of one sequence (the host's plan).
template <int D, int GP, int FMT, bool W16 = false, int QB = 0>
__global__ __launch_bounds__(kThreads, (QB ? QB % 10 : 2)) void sdpa_decode_mfma_ragged_kernel(DecodeDev p, const RaggedItem *__restrict__ items) {
    const RaggedItem it = items[blockIdx.x];
    const int kvh = blockIdx.y;
    MfmaWork wk;
    wk.seq = it.seq, wk.kvh = kvh;
    wk.kbase = it.k + (int64_t)kvh * it.stride_h;
    wk.vbase = it.v + (int64_t)kvh * it.stride_h;
    wk.ksbase = wk.vsbase = nullptr;
    if constexpr (FMT != TROCM_F16) {
        wk.ksbase = it.ks + (int64_t)kvh * it.sc_stride_h;
        wk.vsbase = it.vs + (int64_t)kvh * it.sc_stride_h;
    }
    wk.T = it.T;
    wk.tile_begin = it.tile_begin, wk.tile_end = it.tile_end, wk.tile_step = kWaves;
    wk.skew_period = 0, wk.skew_split = 0;
    wk.nsplit = it.nsplit;
    wk.slot = ((int64_t)it.slot0 + it.split) * p.Hkv + kvh;
    wk.new_pos = p.k_new ? it.T - 1 : -1;
    wk.counter = p.counters ? p.counters + (int64_t)it.seq * p.Hkv + kvh : nullptr;
    wk.part_first = (int64_t)it.slot0 * p.Hkv + kvh, wk.part_stride = p.Hkv;
    wk.mask = nullptr;
    if constexpr (QB / 100 == 9)
        decode_mfma_body<D, GP, FMT, false, W16, true>(p, wk);
    else if constexpr (QB >= 100)
        decode_mfma_qdiag_body<GP, FMT, (QB / 10) % 10, (QB / 100 == 3 || QB / 100 == 5 || QB / 100 == 7 ? 8 : 4), (QB / 100 >= 4), (QB / 100 >= 6)>(p, wk);
    else if constexpr (QB != 0)
        decode_mfma_qblock_body<GP, FMT, QB / 10>(p, wk);
    else
        decode_mfma_body<D, GP, FMT, false, W16>(p, wk);
}

// Up to 16 heads per kv head: the 16-wide tiles (batch 8, 8226 tokens, f16: 49.3 -> 48.5 us; batch 1 15.4 -> 14.5 us;
// Q8_0 at 16384 tokens 57-59 -> 55.5 us, Q4_0 46-48 -> 45 us; three workgroups per CU, which the Q8_0 variant reaches
// at 168 registers, gain nothing: the loop is bound by instruction issue).  TROCM_DECODE_MFMA16 = 0 / 1 / 2 selects
// never / quantised formats only / always.
bool use_16_wide(int fmt) {
    static const int mode = getenv("TROCM_DECODE_MFMA16") ? atoi(getenv("TROCM_DECODE_MFMA16")) : 2;
    return mode == 2 || (mode == 1 && fmt != TROCM_F16);
}

// Quantised caches on the 16-wide tiles: block scales applied outside the products (decode_mfma_qblock_body) unless
// TROCM_DECODE_QBLOCK=0 asks for the kernel that dequantises every element on the way into the LDS tile.
bool use_block_scaling() {
    static const int on = getenv("TROCM_DECODE_QBLOCK") ? atoi(getenv("TROCM_DECODE_QBLOCK")) : 1;
    return on != 0;
}

// The block-scaling kernel keeps one tile (Q8_0) or two (Q4_0: half the bytes per tile) ahead in registers, two
// workgroups per compute unit.  Measured at batch 8, 16384 tokens: a tile more ahead 52.1 -> 54.6 us (Q8_0) and 37.7 ->
// 39.2 us (Q4_0); three workgroups per compute unit (Q4_0, 162 registers) 39.2 us.
// Up to 4 heads per kv head take the diagonal body (decode_mfma_qdiag_body) unless TROCM_DECODE_QDIAG=0.
bool use_diagonal() {
    static const int on = getenv("TROCM_DECODE_QDIAG") ? atoi(getenv("TROCM_DECODE_QDIAG")) : 1;
    return on != 0;
}
// 5..8 heads per kv head: the diagonal body with 8 heads and a pair of blocks across the columns (batch 8, 16384 tokens,
// Q4_0, 8 heads per kv head: 37.8 us on the 16 columns of heads -> 34.2 us) unless TROCM_DECODE_QDIAG_PAIRS=0.  (Two sets
// of four heads in the 4 x 4 arrangement, every unpacked fragment feeding two products, were measured first: 42.2 us,
// the score-side instructions double.)
bool use_diagonal_pairs() {
    static const int on = getenv("TROCM_DECODE_QDIAG_PAIRS") ? atoi(getenv("TROCM_DECODE_QDIAG_PAIRS")) : 1;
    return on != 0;
}
// The diagonal bodies sum a head's blocks with a reduce-scatter over neighbouring lanes and exponentiate each score once
// per head instead of once per block column (batch 8, 16384 tokens, Q4_0: 4 heads per kv head 32.3 -> 30.9 us, 8 heads
// 34.5 -> 33 us; Q8_0 49.3 -> 48.8 us) unless TROCM_DECODE_QDIAG_RS=0.
bool use_diagonal_rs() {
    static const int on = getenv("TROCM_DECODE_QDIAG_RS") ? atoi(getenv("TROCM_DECODE_QDIAG_RS")) : 1;
    return on != 0;
}
template <int GP, int FMT>
void launch_qblock(const DecodeDev &p, dim3 grid, hipStream_t s) {
    if constexpr (GP == 8) {
        if (p.rope_cos) {   // (the caller has asked decode_quant_rotates_in_kernel)
            if (p.g_real <= 4)
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 612 : 622)>), grid, dim3(kThreads), 0, s, p);
            else
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 712 : 722)>), grid, dim3(kThreads), 0, s, p);
            return;
        }
        if (p.g_real <= 4 && use_diagonal()) {
            if (use_diagonal_rs())
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 412 : 422)>), grid, dim3(kThreads), 0, s, p);
            else
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 112 : 122)>), grid, dim3(kThreads), 0, s, p);
            return;
        }
        if (use_diagonal() && use_diagonal_pairs()) {   // 5..8 heads per kv head: 8 heads x a pair of blocks across the columns
            if (use_diagonal_rs())
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 512 : 522)>), grid, dim3(kThreads), 0, s, p);
            else
                hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 312 : 322)>), grid, dim3(kThreads), 0, s, p);
            return;
        }
    }
    hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, GP, FMT, false, true, (FMT == TROCM_Q8_0 ? 12 : 22)>), grid, dim3(kThreads), 0, s, p);
}

template <int D, int GP, int FMT = TROCM_F16>
int launch_gp(const DecodeDev &p, dim3 grid, hipStream_t s) {
    if (FMT == TROCM_F16 && p.rope_cos)   // (the caller has checked: 16-wide tiles, no mask)
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<D, (GP <= 16 ? GP : 16), TROCM_F16, false, true, 902>), grid, dim3(kThreads), 0, s, p);
    else if (FMT == TROCM_F16 && p.mask && GP <= 16 && use_16_wide(FMT))
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<D, (GP <= 16 ? GP : 16), TROCM_F16, true, true>), grid, dim3(kThreads), 0, s, p);
    else if (FMT == TROCM_F16 && p.mask)
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<D, GP, TROCM_F16, true>), grid, dim3(kThreads), 0, s, p);
    else if (FMT != TROCM_F16 && D == 128 && GP <= 16 && use_16_wide(FMT) && use_block_scaling() && p.scale_log2 > 0.0f)
        launch_qblock<(GP <= 16 ? GP : 16), (FMT != TROCM_F16 ? FMT : TROCM_Q8_0)>(p, grid, s);
    else if (GP <= 16 && use_16_wide(FMT))
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<D, (GP <= 16 ? GP : 16), FMT, false, true>), grid, dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<D, GP, FMT>), grid, dim3(kThreads), 0, s, p);
    if (p.nsplit > 1 && p.counters == nullptr)
        hipLaunchKernelGGL((sdpa_decode_merge_kernel<__half, D, GP>), dim3(grid.y, grid.z, p.g_real), dim3(D), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_decode (mfma) launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <int D>
int launch_d(const DecodeDev &p, int gp, dim3 grid, hipStream_t s) {
    switch (gp) {
        case 8: return launch_gp<D, 8>(p, grid, s);
        case 16: return launch_gp<D, 16>(p, grid, s);
        default: return launch_gp<D, 32>(p, grid, s);
    }
}

template <int FMT>
int launch_quant(const DecodeDev &p, int gp, dim3 grid, hipStream_t s) {
    switch (gp) {
        case 8: return launch_gp<128, 8, FMT>(p, grid, s);
        case 16: return launch_gp<128, 16, FMT>(p, grid, s);
        default: return launch_gp<128, 32, FMT>(p, grid, s);
    }
}

template <int D, int GP, int FMT = TROCM_F16>
int launch_ragged_gp(const DecodeDev &p, const RaggedItem *items, int n_items, const RaggedSeqSlots *seqs, int n_seq,
                     bool any_split, hipStream_t s) {
    if (p.rope_cos && FMT == TROCM_F16)   // (the caller has checked: 16-wide tiles)
        hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<D, (GP <= 16 ? GP : 16), TROCM_F16, true, 902>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    else if (p.rope_cos && GP == 8 && p.g_real <= 4)   // (... and decode_quant_rotates_in_kernel)
        hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 622 : 612)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    else if (p.rope_cos && GP == 8)
        hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 722 : 712)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    else if (FMT != TROCM_F16 && D == 128 && GP <= 16 && use_16_wide(FMT) && use_block_scaling() && p.scale_log2 > 0.0f)
        if (GP == 8 && p.g_real <= 4 && use_diagonal() && use_diagonal_rs())
            hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 422 : 412)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
        else if (GP == 8 && p.g_real <= 4 && use_diagonal())
            hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 122 : 112)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
        else if (GP == 8 && use_diagonal() && use_diagonal_pairs() && use_diagonal_rs())
            hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 522 : 512)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
        else if (GP == 8 && use_diagonal() && use_diagonal_pairs())
            hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, 8, (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 322 : 312)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
        else
            hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<128, (GP <= 16 ? GP : 16), (FMT != TROCM_F16 ? FMT : TROCM_Q8_0), true, (FMT == TROCM_Q4_0 ? 22 : 12)>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    else if (GP <= 16 && use_16_wide(FMT))
        hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<D, (GP <= 16 ? GP : 16), FMT, true>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    else
        hipLaunchKernelGGL((sdpa_decode_mfma_ragged_kernel<D, GP, FMT>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    if (any_split && !p.counters)   // with counters the last workgroup of a sequence-head has merged it
        hipLaunchKernelGGL((sdpa_decode_ragged_merge_kernel<__half, D, GP>), dim3(p.Hkv, n_seq, p.g_real), dim3(D), 0, s, p, seqs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("ragged sdpa_decode (mfma) launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <int D>
int launch_ragged_d(const DecodeDev &p, int gp, const RaggedItem *items, int n_items, const RaggedSeqSlots *seqs, int n_seq,
                    bool any_split, hipStream_t s) {
    switch (gp) {
        case 8: return launch_ragged_gp<D, 8>(p, items, n_items, seqs, n_seq, any_split, s);
        case 16: return launch_ragged_gp<D, 16>(p, items, n_items, seqs, n_seq, any_split, s);
        default: return launch_ragged_gp<D, 32>(p, items, n_items, seqs, n_seq, any_split, s);
    }
}

}  // namespace

// Group sizes this formulation takes, and the padded size (rows of the partial records) that runs them.
// One head per kv head is faster on the vector-ALU kernel (batch 8, 8226 tokens: 43.4 against 47.4 us);
// from two heads on this one is (4 heads: 47.1 against 51.5 us, batch 32 159 against 168 us; 8 heads:
// 47 against 88 us).  TROCM_DECODE_MFMA_MIN_GROUP overrides the threshold.
int decode_mfma_group(int64_t g_real) {
    static const int min_group = getenv("TROCM_DECODE_MFMA_MIN_GROUP") ? atoi(getenv("TROCM_DECODE_MFMA_MIN_GROUP")) : 2;
    if (g_real < min_group || g_real > 32) return 0;
    return g_real <= 8 ? 8 : g_real <= 16 ? 16 : 32;
}

template <int FMT>
int launch_ragged_quant(const DecodeDev &p, int gp, const RaggedItem *items, int n_items, const RaggedSeqSlots *seqs, int n_seq,
                        bool any_split, hipStream_t s) {
    switch (gp) {
        case 8: return launch_ragged_gp<128, 8, FMT>(p, items, n_items, seqs, n_seq, any_split, s);
        case 16: return launch_ragged_gp<128, 16, FMT>(p, items, n_items, seqs, n_seq, any_split, s);
        default: return launch_ragged_gp<128, 32, FMT>(p, items, n_items, seqs, n_seq, any_split, s);
    }
}

int launch_sdpa_decode_ragged_mfma(const DecodeDev &p, int kv_fmt, int gp, int64_t D, const RaggedItem *items, int n_items,
                                   const RaggedSeqSlots *seqs, int n_seq, bool any_split, hipStream_t s) {
    if (kv_fmt == TROCM_Q8_0) return launch_ragged_quant<TROCM_Q8_0>(p, gp, items, n_items, seqs, n_seq, any_split, s);
    if (kv_fmt == TROCM_Q4_0) return launch_ragged_quant<TROCM_Q4_0>(p, gp, items, n_items, seqs, n_seq, any_split, s);
    return D == 128 ? launch_ragged_d<128>(p, gp, items, n_items, seqs, n_seq, any_split, s)
                    : launch_ragged_d<64>(p, gp, items, n_items, seqs, n_seq, any_split, s);
}

// Quantised cache planes (the caller has checked formats, alignment and strides and filled p but for the
// splits): 2 = not taken (one head per kv head).
// Whether the launch below would run one of the two bodies that take a step's new token from the step's inputs.
// Whether a step over a quantised cache can rotate q and the new key inside the attention launch: the (head, block) bodies
// with the reduce-scatter, i.e. up to 8 heads per kv head.
bool decode_quant_rotates_in_kernel(int64_t g_real) {
    return g_real >= 2 && g_real <= 8 && decode_mfma_group(g_real) == 8 && use_16_wide(TROCM_Q8_0) && use_block_scaling() && use_diagonal() &&
           use_diagonal_pairs() && use_diagonal_rs();
}

bool decode_quant_appends_in_kernel(int64_t g_real, float scale) {
    static const int on = getenv("TROCM_DECODE_QUANT_FUSED_APPEND") ? atoi(getenv("TROCM_DECODE_QUANT_FUSED_APPEND")) : 1;
    const int gp = decode_mfma_group(g_real);
    return on && gp != 0 && gp <= 16 && use_16_wide(TROCM_Q8_0) && use_block_scaling() && scale > 0.0f;
}

int launch_sdpa_decode_quant_mfma(DecodeDev &p, int kv_fmt, int64_t B, void *workspace, size_t workspace_bytes, hipStream_t s) {
    const int gp = decode_mfma_group(p.g_real);
    if (gp == 0) return 2;
    const int64_t BH = B * p.Hkv;
    const int n_tiles = (p.T + kTile - 1) / kTile;
    static const int wg_per_cu = getenv("TROCM_DECODE_QUANT_WG_PER_CU") ? atoi(getenv("TROCM_DECODE_QUANT_WG_PER_CU")) : 2;
    int nsplit = fit_decode_splits(choose_decode_splits(BH, gp, n_tiles, wg_per_cu), BH, gp, 128, workspace, workspace_bytes);
    const int tps = (n_tiles + nsplit - 1) / nsplit;
    nsplit = (n_tiles + tps - 1) / tps;
    p.tiles_per_split = tps, p.nsplit = nsplit;
    static const int interleave = getenv("TROCM_DECODE_INTERLEAVE") ? atoi(getenv("TROCM_DECODE_INTERLEAVE")) : 1;
    p.interleave = interleave;
    p.live_trim = decode_live_trim();
    p.part_ml = (float *)((char *)workspace + kWsCounterBytes);
    p.part_o = p.part_ml + (size_t)BH * nsplit * 2 * gp;
    static const int tail = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    p.counters = nullptr;
    if (tail && gp <= 8 && nsplit > 1 && nsplit <= kWideMergeMax && BH <= (int64_t)(kWsCounterBytes / sizeof(int))) p.counters = (int *)workspace;
    dim3 grid(nsplit, (unsigned)p.Hkv, (unsigned)B);
    return kv_fmt == TROCM_Q8_0 ? launch_quant<TROCM_Q8_0>(p, gp, grid, s) : launch_quant<TROCM_Q4_0>(p, gp, grid, s);
}

int launch_sdpa_decode_kivi(const KiviSdpaArgs &a, hipStream_t s) {
    if (a.Hq % a.Hkv) return 2;
    const int64_t g_real = a.Hq / a.Hkv;
    const int gp = decode_mfma_group(g_real);
    if (gp == 0 || gp > 16) return 2;
    if (a.T <= 0 || a.T > (1ll << 30) || a.B > 65535 || a.Hkv > 65535 || !(a.scale > 0.0f)) return 2;
    if ((uintptr_t)a.q % 16 || (uintptr_t)a.k_codes % 16 || (uintptr_t)a.v_codes % 16 || (uintptr_t)a.k_chan_scale % 16) return 2;
    const int64_t BH = a.B * a.Hkv;
    const int n_tiles = (int)((a.T + kTile - 1) / kTile);
    int nsplit = fit_decode_splits(choose_decode_splits(BH, gp, n_tiles, 2), BH, gp, 128, a.workspace, a.workspace_bytes);
    const int tps = (n_tiles + nsplit - 1) / nsplit;
    nsplit = (n_tiles + tps - 1) / tps;
    DecodeDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const char *)a.q, p.out = (char *)a.out;
    p.k = (const char *)a.k_codes, p.v = (const char *)a.v_codes;
    if (a.k_cap_rows != a.v_cap_rows) return 2;   // one pair of strides serves both code planes
    p.kv_stride_h = a.k_cap_rows * 128, p.kv_stride_b = a.Hkv * p.kv_stride_h, p.kv_stride_t = 128;
    p.k_scales = (const char *)a.v_tok_scale, p.v_scales = (const char *)a.v_tok_lo;
    p.sc_stride_h = a.v_cap_rows * 4, p.sc_stride_b = a.Hkv * p.sc_stride_h;
    p.chan_scale = a.k_chan_scale;
    p.T = (int)a.T;
    p.tiles_per_split = tps, p.nsplit = nsplit;
    p.Hq = (int)a.Hq, p.Hkv = (int)a.Hkv, p.g_real = (int)g_real;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    p.new_pos = (int)a.T - 1;
    static const int interleave = getenv("TROCM_DECODE_INTERLEAVE") ? atoi(getenv("TROCM_DECODE_INTERLEAVE")) : 1;
    p.interleave = interleave;
    p.live_trim = decode_live_trim();
    p.part_ml = (float *)((char *)a.workspace + kWsCounterBytes);
    p.part_o = p.part_ml + (size_t)BH * nsplit * 2 * gp;
    static const int tail = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    if (tail && gp <= 8 && nsplit > 1 && nsplit <= kWideMergeMax && BH <= (int64_t)(kWsCounterBytes / sizeof(int))) p.counters = (int *)a.workspace;
    dim3 grid(nsplit, (unsigned)a.Hkv, (unsigned)a.B);
    if (gp == 8) {
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, 8, TROCM_Q8_0, false, true, 212>), grid, dim3(kThreads), 0, s, p);
        if (p.nsplit > 1 && p.counters == nullptr)
            hipLaunchKernelGGL((sdpa_decode_merge_kernel<__half, 128, 8>), dim3(grid.y, grid.z, p.g_real), dim3(128), 0, s, p);
    } else {
        hipLaunchKernelGGL((sdpa_decode_mfma_kernel<128, 16, TROCM_Q8_0, false, true, 212>), grid, dim3(kThreads), 0, s, p);
        if (p.nsplit > 1 && p.counters == nullptr)
            hipLaunchKernelGGL((sdpa_decode_merge_kernel<__half, 128, 16>), dim3(grid.y, grid.z, p.g_real), dim3(128), 0, s, p);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_decode (affine u8) launch failed: %s", hipGetErrorString(e));
    return 0;
}

int launch_sdpa_decode_mfma(const SdpaArgs &a, hipStream_t s) {
    if (a.Sq != 1) return 2;
    // mask rows are read by 8-byte loads: [mask_b, mask_h, 1, Sk] with Sk % 4 == 0 (the vector-ALU kernel takes the others)
    if (a.mask && (a.Sk % 4 != 0 || (uintptr_t)a.mask % 8 != 0 || a.k_new != nullptr)) return 2;
    if (a.kv_fmt != TROCM_F16 || a.q_dtype != TROCM_F16) return 2;
    if (a.D != 64 && a.D != 128) return 2;
    if (a.Hq % a.Hkv) return 2;
    const int64_t g_real = a.Hq / a.Hkv;
    const int gp = decode_mfma_group(g_real);
    if (gp == 0) return 2;
    if ((a.kv_stride_b * 2) % 16 || (a.kv_stride_h * 2) % 16 || (a.kv_stride_t * 2) % 16) return 2;
    if ((uintptr_t)a.k % 16 || (uintptr_t)a.v % 16 || (uintptr_t)a.q % 16) return 2;
    if (a.Sk <= 0 || a.Sk > (1ll << 30) || a.kv_stride_t * 2 * kTile >= (1ll << 31)) return 2;
    if (a.B > 65535 || a.Hkv > 65535) return 2;
    const int64_t BH = a.B * a.Hkv;
    const int n_tiles = (int)((a.Sk + kTile - 1) / kTile);
    int nsplit = fit_decode_splits(choose_decode_splits(BH, gp, n_tiles, 1), BH, gp, a.D, a.workspace, a.workspace_bytes);
    const int tps = (n_tiles + nsplit - 1) / nsplit;
    nsplit = (n_tiles + tps - 1) / tps;
    DecodeDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const char *)a.q, p.out = (char *)a.out, p.k = (const char *)a.k, p.v = (const char *)a.v;
    p.kv_stride_b = a.kv_stride_b * 2, p.kv_stride_h = a.kv_stride_h * 2, p.kv_stride_t = a.kv_stride_t * 2;
    p.T = (int)a.Sk;
    p.tiles_per_split = tps, p.nsplit = nsplit;
    p.Hq = (int)a.Hq, p.Hkv = (int)a.Hkv, p.g_real = (int)g_real;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    p.k_new = (const char *)a.k_new, p.v_new = (const char *)a.v_new;
    p.new_pos = a.new_pos >= 0 ? (int)a.new_pos : (int)a.Sk - 1;
    if (p.k_new && (p.v_new == nullptr || (uintptr_t)p.k_new % 16 || (uintptr_t)p.v_new % 16)) return 2;
    if (a.rope_cos) {   // q and k_new rotated on the way in: the 16-wide f16 body only
        if (!a.rope_sin || a.mask || !p.k_new || gp > 16 || !use_16_wide(TROCM_F16)) return 2;
        if ((uintptr_t)a.rope_cos % 16 || (uintptr_t)a.rope_sin % 16 || (a.rope_stride_b * 2) % 16) return 2;
        p.rope_cos = (const char *)a.rope_cos, p.rope_sin = (const char *)a.rope_sin, p.rope_stride_b = a.rope_stride_b * 2;
    }
    p.part_ml = (float *)((char *)a.workspace + kWsCounterBytes);
    p.part_o = p.part_ml + (size_t)BH * nsplit * 2 * gp;
    static const int interleave = getenv("TROCM_DECODE_INTERLEAVE") ? atoi(getenv("TROCM_DECODE_INTERLEAVE")) : 1;
    p.interleave = interleave;
    // Workgroups are handed to the 8 XCDs in turn and the odd XCDs stream about a tenth slower than the even ones
    // (time stamps per workgroup: the tile loops of a launch of equal shares end at 33 - 36 us on XCDs 0, 2, 4, 6 and
    // at 37 - 40 us on 1, 3, 5, 7, whatever the shares' addresses): with an even number of splits the odd splits sit
    // on odd XCDs, and in every 16th round of groups they leave their group to their even neighbour (17 : 15).
    // TROCM_DECODE_XCD_SKEW: the period in rounds, 0 = equal shares.
    static const int xcd_skew = getenv("TROCM_DECODE_XCD_SKEW") ? atoi(getenv("TROCM_DECODE_XCD_SKEW")) : 16;
    p.xcd_skew = xcd_skew;
    p.live_trim = decode_live_trim();
    if (a.mask) {   // [mask_b, mask_h, 1, Sk] dense f16
        p.mask = (const char *)a.mask;
        p.mask_stride_h = a.mask_h > 1 ? a.Sk * 2 : 0;
        p.mask_stride_b = a.mask_b > 1 ? a.mask_h * a.Sk * 2 : 0;
    }
    // The last workgroup to arrive merges the splits, except in a short launch with many splits per sequence-head
    // (one or two sequences over up to 16384 tokens: more than kTailMergeMax partial records per head, merged by
    // one workgroup per kv head): there the merge launch, one workgroup per query head, is the shorter way in
    // spite of the launch gap (batch 1, 8192 tokens: 13.6 us against 14.9 us; batch 2: 18.0 against 19.0; from
    // 32768 tokens or 3 sequences on the two are level or the in-kernel merge wins).  TROCM_DECODE_TAIL_MERGE:
    // 0 = always the launch, 2 = always in the kernel.
    static const int tail = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    const bool short_and_wide = nsplit > kTailMergeMax && a.B <= 2 && a.Sk <= 16384;
    if (tail && (tail == 2 || !short_and_wide) && gp <= 8 && nsplit > 1 && nsplit <= kWideMergeMax && BH <= (int64_t)(kWsCounterBytes / sizeof(int)))
        p.counters = (int *)a.workspace;
    dim3 grid(nsplit, (unsigned)a.Hkv, (unsigned)a.B);
    return a.D == 128 ? launch_d<128>(p, gp, grid, s) : launch_d<64>(p, gp, grid, s);
}

}  // namespace trocm
