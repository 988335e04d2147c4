// KIVI-style affine KV-cache quantisation: tract's storage-quantised cache op and its fused variant.
//
//   QuantizedDynKeyValueCache  transformers/src/ops/quant_dyn_kv_cache.rs:92-250, :334-495
//       Values per token (PerTokenStore), Keys per channel in frozen blocks of 32 tokens
//       (BlockChannelStore), the first 4 "sink" tokens and the partial key block kept in f32,
//       4 or 8 bits per code; the op's output is the whole cache dequantised to the input type.
//   QuantizedKvSdpa            transformers/src/ops/kv_quant.rs:105-236, :242-330
//       u8 codes, Values per token, Keys per channel with RUNNING lo / scale (old codes are read
//       back with the current parameters), followed by non-causal attention over the
//       dequantised cache.
//
// The stored bytes and parameters must equal the CPU op's, so every floating-point step is spelled
// out (this file is compiled with -ffp-contract=off): f32 subtraction, IEEE division, f32::round
// (half away from zero), clamp, saturating `as u8` with NaN -> 0; `lo + code * scale` with two
// roundings.  min / max ignore NaN like f32::min / f32::max (v_min_f32 / v_max_f32 in IEEE mode).
//
// Device layout, one object per tensor, BH = batch * heads rows of everything:
//   sink      [BH, sink_tokens, D] f32
//   codes     [BH, cap_rows, row_bytes] u8, row_bytes = ceil(D * bits / 8) (4 bits: even index -> low nibble)
//   lo, scale per token [BH, cap_rows] / per block and channel [BH, cap_rows / 32, D] / per channel [BH, D]
//   residual  [BH, 32, D] f32 (block layout: the partial block)
// cap_rows doubles (multiples of 32).  All of it is HBM-bound byte work: a token costs its own bytes on
// append, the dequantising read costs row_bytes + 2 or 4 bytes per element.
#include <hip/hip_fp16.h>
#include <new>
#include <type_traits>
#include "common.h"

namespace trocm {
namespace {

constexpr int kKeyBlock = 32;   // quant_dyn_kv_cache.rs:153

__device__ __forceinline__ float ld(const float *p) { return *p; }
// A value on its way into fminf / fmaxf: a signalling NaN is quieted first.  v_min_f32 / v_max_f32 answer NaN for a
// signalling one, and the next operation of the chain, which ignores that NaN, has then lost what came before it;
// f32::min / f32::max skip every NaN alike.
__device__ __forceinline__ float quiet(float x) { return __builtin_canonicalizef(x); }

// Exchanges between lanes on the vector ALU (DPP modifiers and the lane-swap instructions) instead of through the LDS
// crossbar (`__shfl_xor` = ds_bpermute_b32: the per-token ingest spent 14 of its 101 us on eight of those per lane).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
// x of lane (l ^ M) for M = 8, 16, 32 combined with this lane's by OP (min or max): exact partners.
template <int M, typename Op>
__device__ __forceinline__ float xor_combine(float x, Op op) {
    static_assert(M == 8 || M == 16 || M == 32, "lane distances 8, 16, 32");
    if constexpr (M == 8) {
        return op(x, dpp_move<0x128>(x));                       // row_ror:8 within a row of 16 lanes
    } else {   // rows 2k and 2k + 1 (halves of the wave) trade places between the two results: one of them is this lane's own
        unsigned a = __builtin_bit_cast(unsigned, x), b = a;
        asm("" : "+v"(b));   // two registers: the instruction swaps in place, and both results are read
        const auto sw = M == 16 ? __builtin_amdgcn_permlane16_swap(a, b, false, false) : __builtin_amdgcn_permlane32_swap(a, b, false, false);
        unsigned s0 = sw[0], s1 = sw[1];
        asm("" : "+v"(s0), "+v"(s1));   // (this compiler folds op(sw[0], sw[1]) to sw[0] when both operands were one value: the minimum was lost)
        return op(__builtin_bit_cast(float, s0), __builtin_bit_cast(float, s1));
    }
}
// Minimum and maximum over aligned groups of N lanes (8, 16, 32, 64), left in every lane of the group.  (Any order of
// exchanges gives the same bits: both are exact.)  Quads, halves of a row and rows by DPP, then pairs of rows, then the
// two halves of the wave.
template <int N>
__device__ __forceinline__ void group_min_max(float &lo, float &hi) {
    static_assert(N == 8 || N == 16 || N == 32 || N == 64, "groups of 8, 16, 32 or 64 lanes");
    auto mn = [](float a, float b) { return fminf(a, b); };
    auto mx = [](float a, float b) { return fmaxf(a, b); };
    lo = fminf(lo, dpp_move<0xB1>(lo)), hi = fmaxf(hi, dpp_move<0xB1>(hi));       // quad_perm [1,0,3,2]
    lo = fminf(lo, dpp_move<0x4E>(lo)), hi = fmaxf(hi, dpp_move<0x4E>(hi));       // quad_perm [2,3,0,1]
    lo = fminf(lo, dpp_move<0x141>(lo)), hi = fmaxf(hi, dpp_move<0x141>(hi));     // row_half_mirror: the other quad of 8 lanes
    if constexpr (N >= 16) lo = fminf(lo, dpp_move<0x140>(lo)), hi = fmaxf(hi, dpp_move<0x140>(hi));   // row_mirror: the other half of the row
    if constexpr (N >= 32) lo = xor_combine<16>(lo, mn), hi = xor_combine<16>(hi, mx);
    if constexpr (N >= 64) lo = xor_combine<32>(lo, mn), hi = xor_combine<32>(hi, mx);
}
__device__ __forceinline__ float ld(const __half *p) { return __half2float(*p); }

// f32 -> f16 as its own instruction: without the barrier the compiler may fold the preceding multiply and add
// into one mixed-precision fma, which rounds once where the CPU op rounds three times.
__device__ __forceinline__ void st(float *p, float x) { *p = x; }
__device__ __forceinline__ void st(__half *p, float x) {
    asm volatile("" : "+v"(x));
    *p = __float2half_rn(x);
}

// f32::round(): half away from zero, as trunc(x + copysign(0.49999997, x)) (the float below 0.5; the sum rounds to
// nearest even, so an exact half ties up to the integer and anything less stays below it; exact for every float,
// checked exhaustively on the host for the exponents where it matters; inf and NaN pass through).
__device__ __forceinline__ float round_half_away(float x) {
    return truncf(__fadd_rn(x, __builtin_copysignf(0.49999997f, x)));
}

// ((x - lo) / scale).round().clamp(0.0, lv) as u8   (quant_dyn_kv_cache.rs:128, :190; kv_quant.rs:110, :219)
__device__ __forceinline__ uint32_t affine_code(float x, float lo, float scale, float lv) {
    float q = round_half_away(__fdiv_rn(__fsub_rn(x, lo), scale));
    if (!(q == q)) return 0;            // clamp keeps NaN, the cast turns it into 0
    q = q < 0.0f ? 0.0f : (q > lv ? lv : q);
    return (uint32_t)q;
}
__device__ __forceinline__ float affine_scale(float lo, float hi, float lv) {   // :127, :186
    return hi > lo ? __fdiv_rn(__fsub_rn(hi, lo), lv) : 1.0f;
}

// The same codes without a division per element.  With inv = RN(1 / scale) the product q0 = RN((x - lo) * inv) lies
// within 2^-22 relative of the reference's quotient q = RN((x - lo) / scale) (three roundings of 2^-24 between them),
// i.e. within 2^-14 absolute wherever a rounding decision is still open (q below lv + 1/2 <= 255.5; from there on
// both clamp to lv, and every negative quotient rounds to a code of 0).  So when the fraction of q0 is at least 2^-13
// away from one half, trunc(q0 + 0.49999997) is the reference's round(q) (see round_half_away); otherwise, and for a
// scale whose reciprocal is not an ordinary float, the eight codes are computed again with the division.  NaN gives 0
// and +inf gives lv on both paths.
__device__ __forceinline__ float affine_inv(float scale) {   // 0: do not use the product
    return (scale >= 0x1p-100f && scale <= 0x1p100f) ? __fdiv_rn(1.0f, scale) : 0.0f;
}
__device__ __forceinline__ int cvt_i32_rz_sat(float x) {   // truncates, saturates, NaN -> 0 (a C cast may assume the value is in range)
    int r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}
// KNOWN: the caller keeps track of whether every inv is usable (non-zero) and passes it as `all_usable` (a walk whose
// parameters change rarely: the 8 comparisons per token leave its loop).
template <bool KNOWN = false, typename Params>   // Params: float (one group for the 8 values) or float[8] (a group per value)
__device__ __forceinline__ void affine_codes8(const float (&x)[8], const Params &lo, const Params &scale, const Params &inv, float lv,
                                              uint32_t (&code)[8], bool all_usable = true) {
    auto at = [](const Params &p, int e) -> float {
        if constexpr (std::is_same<Params, float>::value) return p;
        else return p[e];
    };
    float near = 1.0f;   // the smallest distance of a fraction from one half (fminf drops a NaN)
    bool usable = all_usable;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float q0 = __fmul_rn(__fsub_rn(x[e], at(lo, e)), at(inv, e));
        near = fminf(near, fabsf(__fsub_rn(__builtin_amdgcn_fractf(q0), 0.5f)));
        code[e] = (uint32_t)max(0, min((int)lv, cvt_i32_rz_sat(__fadd_rn(q0, 0.49999997f))));
        if constexpr (!KNOWN) usable = usable && at(inv, e) != 0.0f;
    }
    if (!(usable && near >= 0x1p-13f)) {
#pragma unroll
        for (int e = 0; e < 8; e++) code[e] = affine_code(x[e], at(lo, e), at(scale, e), lv);
    }
}

// The same for 8-bit codes, as the two words a row stores for the 8 values: v_cvt_pk_u8_f32 rounds to the nearest integer
// (ties to even), saturates to [0, 255], turns a NaN into 0 and puts the byte in its place -- the reference's
// round-half-away and clamp wherever the fraction is not one half, which is exactly what the re-check excludes -- so
// the product needs neither the add and truncation nor the clamp nor the shifts that pack the bytes.
template <bool KNOWN = false, typename Params>
__device__ __forceinline__ void affine_words8_u8(const float (&x)[8], const Params &lo, const Params &scale, const Params &inv,
                                                 uint32_t &w0, uint32_t &w1, bool all_usable = true) {
    auto at = [](const Params &p, int e) -> float {
        if constexpr (std::is_same<Params, float>::value) return p;
        else return p[e];
    };
    float near = 1.0f;
    bool usable = all_usable;
    w0 = 0, w1 = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float q0 = __fmul_rn(__fsub_rn(x[e], at(lo, e)), at(inv, e));
        near = fminf(near, fabsf(__fsub_rn(__builtin_amdgcn_fractf(q0), 0.5f)));
        if (e < 4) w0 = __builtin_amdgcn_cvt_pk_u8_f32(q0, e, w0);
        else w1 = __builtin_amdgcn_cvt_pk_u8_f32(q0, e - 4, w1);
        if constexpr (!KNOWN) usable = usable && at(inv, e) != 0.0f;
    }
    if (!(usable && near >= 0x1p-13f)) {
        uint32_t code[8];
#pragma unroll
        for (int e = 0; e < 8; e++) code[e] = affine_code(x[e], at(lo, e), at(scale, e), 255.0f);
        w0 = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
        w1 = code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24);
    }
}

// dst[bh][dst_t0 + i][c] = (f32) src[bh][src_t0 + i][c], i < n: sink tokens and the partial key block.
template <typename SrcT>
__global__ void kivi_rows_to_f32_kernel(const SrcT *__restrict__ src, int64_t S, int64_t src_t0, float *__restrict__ dst,
                                        int64_t dst_pitch, int64_t dst_t0, int n, int D) {
    const int bh = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * D) return;
    const int i = e / D, c = e - i * D;
    dst[((int64_t)bh * dst_pitch + dst_t0 + i) * D + c] = ld(src + ((int64_t)bh * S + src_t0 + i) * D + c);
}

// Values, one wave per (head row, token): lo / hi over the token's D channels, then its codes (PerTokenStore::push_token).
template <typename SrcT, int BITS>
__global__ void __launch_bounds__(256) kivi_quant_tokens_kernel(const SrcT *__restrict__ src, int64_t S, int64_t src_t0, int n, int D,
                                                                uint8_t *__restrict__ codes, int64_t cap_rows, int row_bytes,
                                                                int64_t row0, float *__restrict__ lo_out, float *__restrict__ scale_out) {
    const int bh = blockIdx.y;
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (i >= n) return;
    const SrcT *row = src + ((int64_t)bh * S + src_t0 + i) * D;
    float lo = INFINITY, hi = -INFINITY;
    for (int c = lane; c < D; c += 64) {
        const float v = ld(row + c);
        lo = fminf(lo, quiet(v));
        hi = fmaxf(hi, quiet(v));
    }
    group_min_max<64>(lo, hi);
    constexpr float lv = (float)((1u << BITS) - 1u);
    const float scale = affine_scale(lo, hi, lv);
    uint8_t *out = codes + ((int64_t)bh * cap_rows + row0 + i) * row_bytes;
    for (int u = lane; u < row_bytes; u += 64) {
        uint32_t byte;
        if (BITS == 8) {
            byte = affine_code(ld(row + u), lo, scale, lv);
        } else {
            const int c0 = 2 * u, c1 = 2 * u + 1;
            byte = affine_code(ld(row + c0), lo, scale, lv) & 15u;
            if (c1 < D) byte |= (affine_code(ld(row + c1), lo, scale, lv) & 15u) << 4;
        }
        out[u] = (uint8_t)byte;
    }
    if (lane == 0) {
        lo_out[(int64_t)bh * cap_rows + row0 + i] = lo;
        scale_out[(int64_t)bh * cap_rows + row0 + i] = scale;
    }
}

// Keys, one workgroup per (block that becomes full, head row), a thread per byte column of the rows: lo / hi of its
// channel(s) over the block's 32 tokens, the frozen parameters, then the 32 codes (BlockChannelStore::finalize_block).
// Row k of the run of blocks comes from the partial block when k < n_res_old, else from the new tokens.
template <typename SrcT, int BITS>
__global__ void __launch_bounds__(256) kivi_finalize_blocks_kernel(const SrcT *__restrict__ src, int64_t S, int64_t src_t0,
                                                                   const float *__restrict__ residual, int n_res_old, int D,
                                                                   uint8_t *__restrict__ codes, int64_t cap_rows, int row_bytes,
                                                                   int64_t row0, float *__restrict__ lo_out, float *__restrict__ scale_out) {
    const int j = blockIdx.x, bh = blockIdx.y;
    constexpr float lv = (float)((1u << BITS) - 1u);
    constexpr int CH = BITS == 8 ? 1 : 2;
    const int64_t blk = row0 / kKeyBlock + j;
    const float *res = residual + (int64_t)bh * kKeyBlock * D;
    const SrcT *fresh = src + ((int64_t)bh * S + src_t0 - n_res_old) * D;   // row k >= n_res_old of the run sits at fresh + k * D
    for (int u = threadIdx.x; u < row_bytes; u += blockDim.x) {
        float lo[CH], scale[CH];
#pragma unroll
        for (int h = 0; h < CH; h++) {
            const int c = CH * u + h;
            float l = INFINITY, hi = -INFINITY;
            if (c < D) {
#pragma unroll 4
                for (int r = 0; r < kKeyBlock; r++) {
                    const int k = j * kKeyBlock + r;
                    const float x = k < n_res_old ? res[(int64_t)k * D + c] : ld(fresh + (int64_t)k * D + c);
                    l = fminf(l, quiet(x));
                    hi = fmaxf(hi, quiet(x));
                }
                const int64_t at = ((int64_t)bh * (cap_rows / kKeyBlock) + blk) * D + c;
                lo_out[at] = l;
                scale_out[at] = affine_scale(l, hi, lv);
            }
            lo[h] = l;
            scale[h] = affine_scale(l, hi, lv);
        }
        // second pass over the block's rows (they are in the cache now): the codes
#pragma unroll 2
        for (int r = 0; r < kKeyBlock; r++) {
            const int k = j * kKeyBlock + r;
            uint32_t byte = 0;
#pragma unroll
            for (int h = 0; h < CH; h++) {
                const int c = CH * u + h;
                if (c < D) {
                    const float x = k < n_res_old ? res[(int64_t)k * D + c] : ld(fresh + (int64_t)k * D + c);
                    const uint32_t code = affine_code(x, lo[h], scale[h], lv);
                    byte |= CH == 1 ? code : (code & 15u) << (4 * h);
                }
            }
            codes[((int64_t)bh * cap_rows + row0 + k) * row_bytes + u] = (uint8_t)byte;
        }
    }
}

// Keys with running parameters, a thread per (head row, channel), tokens in order (QuantKeyCache::push_token):
// lo follows the minimum, scale only grows, each token is coded under the parameters current at its push.
template <typename SrcT>
__global__ void kivi_running_push_kernel(const SrcT *__restrict__ src, int64_t S, int n, int D, uint8_t *__restrict__ codes,
                                         int64_t cap_rows, int64_t row0, float *__restrict__ lo_io, float *__restrict__ scale_io) {
    const int bh = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = lo_io[(int64_t)bh * D + c], scale = scale_io[(int64_t)bh * D + c];
    for (int t = 0; t < n; t++) {
        const float val = ld(src + ((int64_t)bh * S + t) * D + c);
        if (val < lo) lo = val;
        const float range = __fsub_rn(val, lo);
        if (range > 0.0f) {
            const float ns = __fdiv_rn(range, 255.0f);
            if (ns > scale) scale = ns;
        }
        codes[((int64_t)bh * cap_rows + row0 + t) * D + c] = (uint8_t)affine_code(val, lo, scale, 255.0f);
    }
    lo_io[(int64_t)bh * D + c] = lo;
    scale_io[(int64_t)bh * D + c] = scale;
}

// The same push for a long run of tokens (a prompt), in chunks of kRunChunk tokens that are scanned side by side.
// The running parameters are prefix results: lo after token t is the first minimal value among lo_before and the tokens
// up to t (`val < lo` never takes a NaN and keeps the earlier of two equal values), scale after token t is the largest
// of scale_before and (val_s - lo_s) / 255 over the tokens s <= t whose range is positive.  Three passes over the
// chunks with two short scans over the chunk results between them give every token the parameters the token-by-token
// loop would have had at its push.
constexpr int kRunChunk = 64;

// pass 1: first minimal value of each chunk and channel (+inf for a chunk of NaNs)
template <typename SrcT>
__global__ void kivi_run_chunk_min_kernel(const SrcT *__restrict__ src, int64_t S, int n, int D, int n_chunks, float *__restrict__ cmin) {
    const int bh = blockIdx.z, k = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = INFINITY;
    const int t1 = min(n, (k + 1) * kRunChunk);
    for (int t = k * kRunChunk; t < t1; t++) {
        const float val = ld(src + ((int64_t)bh * S + t) * D + c);
        if (val < lo) lo = val;
    }
    cmin[((int64_t)bh * n_chunks + k) * D + c] = lo;
}
// scan 1: lo at the start of every chunk (in place), and the final lo into the store.  Sixteen chunk results are
// requested together: one dependent load per chunk made this a chain of memory latencies (32 us for 128 chunks).
__global__ void kivi_run_scan_min_kernel(float *__restrict__ cmin, int D, int n_chunks, float *__restrict__ lo_io) {
    const int bh = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = lo_io[(int64_t)bh * D + c];
    float *col = cmin + (int64_t)bh * n_chunks * D + c;
    for (int k0 = 0; k0 < n_chunks; k0 += 16) {
        float m[16];
#pragma unroll
        for (int i = 0; i < 16; i++) m[i] = k0 + i < n_chunks ? col[(int64_t)(k0 + i) * D] : INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (k0 + i < n_chunks) col[(int64_t)(k0 + i) * D] = lo;
            if (m[i] < lo) lo = m[i];
        }
    }
    lo_io[(int64_t)bh * D + c] = lo;
}
// pass 2: the largest scale candidate of each chunk and channel (0 when no token of the chunk has a positive range)
template <typename SrcT>
__global__ void kivi_run_chunk_scale_kernel(const SrcT *__restrict__ src, int64_t S, int n, int D, int n_chunks,
                                            const float *__restrict__ lo_start, float *__restrict__ cmax) {
    const int bh = blockIdx.z, k = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = lo_start[((int64_t)bh * n_chunks + k) * D + c], best = 0.0f;
    const int t1 = min(n, (k + 1) * kRunChunk);
    for (int t = k * kRunChunk; t < t1; t++) {
        const float val = ld(src + ((int64_t)bh * S + t) * D + c);
        if (val < lo) lo = val;
        const float range = __fsub_rn(val, lo);
        if (range > 0.0f) {
            const float ns = __fdiv_rn(range, 255.0f);
            if (ns > best) best = ns;
        }
    }
    cmax[((int64_t)bh * n_chunks + k) * D + c] = best;
}
// scan 2: scale at the start of every chunk (in place), and the final scale into the store
__global__ void kivi_run_scan_scale_kernel(float *__restrict__ cmax, int D, int n_chunks, float *__restrict__ scale_io) {
    const int bh = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float scale = scale_io[(int64_t)bh * D + c];
    float *col = cmax + (int64_t)bh * n_chunks * D + c;
    for (int k0 = 0; k0 < n_chunks; k0 += 16) {
        float m[16];
#pragma unroll
        for (int i = 0; i < 16; i++) m[i] = k0 + i < n_chunks ? col[(int64_t)(k0 + i) * D] : 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (k0 + i < n_chunks) col[(int64_t)(k0 + i) * D] = scale;
            if (m[i] > scale) scale = m[i];
        }
    }
    scale_io[(int64_t)bh * D + c] = scale;
}
// The 128-bit path makes one pass for both scans.  Per chunk and channel it leaves the first minimal value (`cmin`), the
// largest value (`cmax`) and the widest range against the chunk's own running minimum (`cown`).  A token's range is
// taken against the smaller of the incoming lo and the chunk's running minimum, i.e. it is the LARGER of RN(x - lo_in)
// and RN(x - own minimum) (the subtraction grows as what is subtracted shrinks), so the chunk's widest range is
// max(RN(cmax - lo_in), cown), its largest scale candidate RN(that / 255), and both running parameters of every chunk's
// start come out of one walk over the chunks.  NaN values take part in nothing (every comparison with them is false),
// exactly as in the token-by-token loop.  In place: cmin becomes the chunk's starting lo, cmax its starting scale.
__global__ void kivi_run_scan_both_kernel(float *__restrict__ cmin, float *__restrict__ cmax, const float *__restrict__ cown, int D,
                                          int n_chunks, float *__restrict__ lo_io, float *__restrict__ scale_io) {
    const int bh = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = lo_io[(int64_t)bh * D + c];
    const float scale0 = scale_io[(int64_t)bh * D + c];
    // The walk carries the widest RANGE so far, not the scale: the quotient by 255 grows with the range, so the largest
    // quotient is the quotient of the widest range, and the divisions (one per chunk, for the scale its tokens start
    // from) stay off the chain from chunk to chunk, which is a subtraction and two comparisons.  Sixteen chunks'
    // results are in registers while the next sixteen are on their way.
    float widest = 0.0f;
    const int64_t base = (int64_t)bh * n_chunks * D + c;
    constexpr int G = 16;
    // (Whole groups of sixteen without a condition anywhere: a load or a store behind a condition becomes a branch, and the
    // compiler then waits for every load where the paths meet.  The prefetch past the last group reads the last chunk again.)
    float mn[2][G], mx[2][G], own[2][G];
    auto load = [&](int k0, float (&a)[G], float (&b)[G], float (&o)[G]) {
#pragma unroll
        for (int i = 0; i < G; i++) {
            const int64_t at = base + (int64_t)min(k0 + i, n_chunks - 1) * D;
            a[i] = cmin[at], b[i] = cmax[at], o[i] = cown[at];
        }
    };
    auto step = [&](float a, float b, float o, float &lo_in, float &w_in) {
        lo_in = lo, w_in = widest;
        const float r = __fsub_rn(b, lo);           // the chunk's largest value against the incoming lo
        widest = r > widest ? r : widest;           // (a NaN range is never wider)
        widest = o > widest ? o : widest;
        lo = a < lo ? a : lo;
    };
    auto start_scale = [&](float w_in) {
        const float ns = w_in > 0.0f ? __fdiv_rn(w_in, 255.0f) : 0.0f;
        return ns > scale0 ? ns : scale0;
    };
    auto walk = [&](int k0, const float (&a)[G], const float (&b)[G], const float (&o)[G]) {
        float lo_in[G], w_in[G];
#pragma unroll
        for (int i = 0; i < G; i++) step(a[i], b[i], o[i], lo_in[i], w_in[i]);
#pragma unroll
        for (int i = 0; i < G; i++) {
            const int64_t at = base + (int64_t)(k0 + i) * D;
            cmin[at] = lo_in[i], cmax[at] = start_scale(w_in[i]);
        }
    };
    const int whole = n_chunks / G * G;
    int k0 = 0;
    if (whole > 0) load(0, mn[0], mx[0], own[0]);
    for (; k0 + 2 * G <= whole; k0 += 2 * G) {
        load(k0 + G, mn[1], mx[1], own[1]);
        walk(k0, mn[0], mx[0], own[0]);
        load(k0 + 2 * G, mn[0], mx[0], own[0]);
        walk(k0 + G, mn[1], mx[1], own[1]);
    }
    if (k0 < whole) walk(k0, mn[0], mx[0], own[0]), k0 += G;
    for (; k0 < n_chunks; k0++) {   // the chunks past the last whole group
        const int64_t at = base + (int64_t)k0 * D;
        float lo_in, w_in;
        step(cmin[at], cmax[at], cown[at], lo_in, w_in);
        cmin[at] = lo_in, cmax[at] = start_scale(w_in);
    }
    lo_io[(int64_t)bh * D + c] = lo;
    const float ns = widest > 0.0f ? __fdiv_rn(widest, 255.0f) : 0.0f;
    scale_io[(int64_t)bh * D + c] = ns > scale0 ? ns : scale0;
}
// pass 3: the codes, every chunk starting from its own parameters
template <typename SrcT>
__global__ void kivi_run_chunk_codes_kernel(const SrcT *__restrict__ src, int64_t S, int n, int D, int n_chunks,
                                            const float *__restrict__ lo_start, const float *__restrict__ scale_start,
                                            uint8_t *__restrict__ codes, int64_t cap_rows, int64_t row0) {
    const int bh = blockIdx.z, k = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= D) return;
    float lo = lo_start[((int64_t)bh * n_chunks + k) * D + c], scale = scale_start[((int64_t)bh * n_chunks + k) * D + c];
    const int t1 = min(n, (k + 1) * kRunChunk);
    for (int t = k * kRunChunk; t < t1; t++) {
        const float val = ld(src + ((int64_t)bh * S + t) * D + c);
        if (val < lo) lo = val;
        const float range = __fsub_rn(val, lo);
        if (range > 0.0f) {
            const float ns = __fdiv_rn(range, 255.0f);
            if (ns > scale) scale = ns;
        }
        codes[((int64_t)bh * cap_rows + row0 + t) * D + c] = (uint8_t)affine_code(val, lo, scale, 255.0f);
    }
}

// ---- the same three steps for head sizes that are a multiple of 8 (and, for the two quantising kernels, 64, 128,
// ---- 256 or 512 with 16-byte aligned sources): a lane owns 8 consecutive channels, so rows move as 128-bit words
struct F8 {
    float v[8];
};
__device__ __forceinline__ F8 ld8(const float *p) {
    const float4 a = reinterpret_cast<const float4 *>(p)[0], b = reinterpret_cast<const float4 *>(p)[1];
    return F8{{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w}};
}
__device__ __forceinline__ F8 ld8(const __half *p) {
    const uint4 w = *reinterpret_cast<const uint4 *>(p);
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
    F8 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        r.v[2 * i] = __half2float(__ushort_as_half((unsigned short)(u[i] & 0xffffu)));
        r.v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(u[i] >> 16)));
    }
    return r;
}
__device__ __forceinline__ void st8(float *p, const F8 &x) {
    reinterpret_cast<float4 *>(p)[0] = make_float4(x.v[0], x.v[1], x.v[2], x.v[3]);
    reinterpret_cast<float4 *>(p)[1] = make_float4(x.v[4], x.v[5], x.v[6], x.v[7]);
}
__device__ __forceinline__ void st8(__half *p, const F8 &x) {
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float a = x.v[2 * i], b = x.v[2 * i + 1];
        asm volatile("" : "+v"(a), "+v"(b));   // conversions stay their own instructions (see st)
        u[i] = (uint32_t)__half_as_ushort(__float2half_rn(a)) | ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
    }
    *reinterpret_cast<uint4 *>(p) = make_uint4(u[0], u[1], u[2], u[3]);
}
// streaming stores for the dequantised cache (written once, read by the next kernel from HBM anyway)
__device__ __forceinline__ void st8_stream(float *p, const F8 &x) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(f32x4{x.v[0], x.v[1], x.v[2], x.v[3]}, reinterpret_cast<f32x4 *>(p));
    __builtin_nontemporal_store(f32x4{x.v[4], x.v[5], x.v[6], x.v[7]}, reinterpret_cast<f32x4 *>(p) + 1);
}
__device__ __forceinline__ void st8_stream(__half *p, const F8 &x) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float a = x.v[2 * i], b = x.v[2 * i + 1];
        asm volatile("" : "+v"(a), "+v"(b));
        u[i] = (uint32_t)__half_as_ushort(__float2half_rn(a)) | ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
    }
    __builtin_nontemporal_store(u32x4{u[0], u[1], u[2], u[3]}, reinterpret_cast<u32x4 *>(p));
}
// 8 codes of one lane's channels packed as the row stores them: 8 bytes, or 4 bytes of nibble pairs (even index low).
template <int BITS>
__device__ __forceinline__ void store_codes8(uint8_t *row, int sub, const uint32_t (&code)[8]) {
    if (BITS == 8) {
        const uint32_t w0 = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
        const uint32_t w1 = code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24);
        *reinterpret_cast<uint2 *>(row + sub * 8) = make_uint2(w0, w1);
    } else {
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) w |= (code[i] & 15u) << (4 * i);
        *reinterpret_cast<uint32_t *>(row + sub * 4) = w;
    }
}

// Eight consecutive channels as they lie in memory (the conversion to f32 happens when the row is used).
struct RawF32x8 { float4 a, b; };
__device__ __forceinline__ RawF32x8 ld8raw(const float *p) { return RawF32x8{reinterpret_cast<const float4 *>(p)[0], reinterpret_cast<const float4 *>(p)[1]}; }
__device__ __forceinline__ uint4 ld8raw(const __half *p) { return *reinterpret_cast<const uint4 *>(p); }
__device__ __forceinline__ F8 cvt8(const RawF32x8 &r) { return F8{{r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w}}; }
__device__ __forceinline__ F8 cvt8(const uint4 &w) {
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
    F8 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        r.v[2 * i] = __half2float(__ushort_as_half((unsigned short)(u[i] & 0xffffu)));
        r.v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(u[i] >> 16)));
    }
    return r;
}

__device__ __forceinline__ void settle(RawF32x8 &r) { asm volatile("" : "+v"(r.a.x), "+v"(r.a.y), "+v"(r.a.z), "+v"(r.a.w), "+v"(r.b.x), "+v"(r.b.y), "+v"(r.b.z), "+v"(r.b.w)); }
__device__ __forceinline__ void settle(uint4 &w) { asm volatile("" : "+v"(w.x), "+v"(w.y), "+v"(w.z), "+v"(w.w)); }

// The three chunk passes of the running Key store for head sizes 64 / 128 / 256 / 512 and 16-byte aligned sources: a lane
// owns 8 consecutive channels of one chunk and walks the chunk's tokens with 128-bit loads; LPR = D / 8 lanes cover a row,
// 256 / LPR chunks share a workgroup.  PASS 1: first minimal value per chunk and channel into `a`; PASS 2: largest scale
// candidate into `b`, starting from the chunk's lo in `a`; PASS 3: the codes, starting from the parameters in `a`, `b`.
// Arithmetic, order and tie-breaking are those of kivi_run_chunk_{min,scale,codes}_kernel.
template <typename SrcT, int LPR, int PASS>
__global__ void __launch_bounds__(256) kivi_run_chunk_vec_kernel(const SrcT *__restrict__ src, int64_t S, int n, int n_chunks,
                                                                 float *__restrict__ a, float *__restrict__ b,
                                                                 uint8_t *__restrict__ codes, int64_t cap_rows, int64_t row0,
                                                                 float *__restrict__ c3 = nullptr) {
    constexpr int D = LPR * 8, CPW = 256 / LPR;
    const int bh = blockIdx.y, k = blockIdx.x * CPW + (int)threadIdx.x / LPR, sub = (int)threadIdx.x % LPR;
    if (k >= n_chunks) return;
    const int64_t at = ((int64_t)bh * n_chunks + k) * D + sub * 8;
    const int t0 = k * kRunChunk, t1 = min(n, t0 + kRunChunk);
    const SrcT *row = src + ((int64_t)bh * S + t0) * D + sub * 8;
    // PASS 3 takes the chunk's rows in groups of 8.  Loads and stores share a counter and are not ordered against each
    // other, so a wait for a row with a store outstanding is a wait for all memory traffic: with the loads of just the
    // tokens at hand and a store per token, every token paid a whole trip to memory (69 us).  Now the next group is
    // requested first, this group's codes are formed into registers, the next group's rows are waited for while only
    // loads (8 tokens old) are outstanding, and then this group's codes are stored: they have the next group's
    // arithmetic to complete in.  (The passes that only load count their loads and are better off without the groups:
    // 31 against 35 us.)  Rows past the chunk's end: its last row again.
    constexpr int G = 8;
    uint32_t cw0[G], cw1[G];   // PASS 3: the group's codes, 8 per token
    auto for_each_token = [&](auto &&body) {
        if constexpr (PASS != 3) {
#pragma unroll 4
            for (int t = t0; t < t1; t++) body(t, ld8(row + (int64_t)(t - t0) * D), 0);
            return;
        }
        auto fetch = [&](int t) { return ld8raw(row + (int64_t)(min(t, t1 - 1) - t0) * D); };
        decltype(fetch(0)) cur[G], nxt[G];
#pragma unroll
        for (int u = 0; u < G; u++) cur[u] = fetch(t0 + u);
        for (int tg = t0; tg < t1; tg += G) {
#pragma unroll
            for (int u = 0; u < G; u++) nxt[u] = fetch(tg + G + u);
#pragma unroll
            for (int u = 0; u < G; u++)
                if (tg + u < t1) body(tg + u, cvt8(cur[u]), u);
#pragma unroll
            for (int u = 0; u < G; u++) settle(nxt[u]), cur[u] = nxt[u];
#pragma unroll
            for (int u = 0; u < G; u++)
                if (tg + u < t1)
                    *reinterpret_cast<uint2 *>(codes + ((int64_t)bh * cap_rows + row0 + tg + u) * D + sub * 8) = make_uint2(cw0[u], cw1[u]);
        }
    };
    if constexpr (PASS == 12) {   // one pass for both scans (kivi_run_scan_both_kernel): first minimum, maximum, widest own range
        F8 mn, mx, own;
#pragma unroll
        for (int e = 0; e < 8; e++) mn.v[e] = INFINITY, mx.v[e] = -INFINITY, own.v[e] = 0.0f;
        for_each_token([&](int, const F8 &x, int) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float val = x.v[e];
                mn.v[e] = val < mn.v[e] ? val : mn.v[e];
                mx.v[e] = val > mx.v[e] ? val : mx.v[e];
                const float range = __fsub_rn(val, mn.v[e]);
                own.v[e] = range > own.v[e] ? range : own.v[e];   // (a NaN range is never wider)
            }
        });
        st8(a + at, mn), st8(b + at, mx), st8(c3 + at, own);
        return;
    }
    F8 lo, sc;
    if (PASS == 1) {
#pragma unroll
        for (int e = 0; e < 8; e++) lo.v[e] = INFINITY;
    } else {
        lo = ld8(a + at);
    }
    if (PASS == 2) {
#pragma unroll
        for (int e = 0; e < 8; e++) sc.v[e] = 0.0f;
    } else if (PASS == 3) {
        sc = ld8(b + at);
    }
    // A channel's scale is the largest RN(range / 255) so far, and that quotient grows with the range.  PASS 2 therefore
    // keeps the widest range of the chunk (compare and select, no branch) and divides once at the end: the same value as
    // the largest of the tokens' quotients.  PASS 3 needs the scale token by token, but only a range wider than any before
    // it can move it, and none below 254.9 times the incoming scale can (its quotient is below that scale): `widest`
    // starts there, and the division sits behind one branch per token that is taken when some lane of the wave has such
    // a range in one of its 8 channels -- rarely, once the first tokens of the sequence have set the scale.  The codes
    // take the reciprocal of the scale with its re-check (affine_codes8), refreshed when the scale moves.
    float widest[8];
    F8 inv;
    bool inv_usable = true;   // every inv is non-zero (kept up to date where a scale moves)
#pragma unroll
    for (int e = 0; e < 8; e++) {
        widest[e] = PASS == 3 ? sc.v[e] * 254.9f : 0.0f;
        inv.v[e] = PASS == 3 ? affine_inv(sc.v[e]) : 0.0f;
        inv_usable = inv_usable && inv.v[e] != 0.0f;
    }
    for_each_token([&](int, const F8 &x, int u) {
        bool wider = false;
        float range[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float val = x.v[e];
            lo.v[e] = val < lo.v[e] ? val : lo.v[e];
            if (PASS >= 2) {
                range[e] = __fsub_rn(val, lo.v[e]);
                if (PASS == 2) widest[e] = range[e] > widest[e] ? range[e] : widest[e];   // (a NaN range is never wider)
                else wider = wider || range[e] > widest[e];
            }
        }
        if (PASS == 3) {
            if (__builtin_amdgcn_ballot_w64(wider) != 0) {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (range[e] > widest[e]) {
                        widest[e] = range[e];
                        const float ns = __fdiv_rn(range[e], 255.0f);
                        if (ns > sc.v[e]) {
                            sc.v[e] = ns;
                            inv.v[e] = affine_inv(ns);
                        }
                    }
                inv_usable = true;
#pragma unroll
                for (int e = 0; e < 8; e++) inv_usable = inv_usable && inv.v[e] != 0.0f;
            }
            affine_words8_u8<true>(x.v, lo.v, sc.v, inv.v, cw0[u], cw1[u], inv_usable);
        }
    });
    if (PASS == 2) {
#pragma unroll
        for (int e = 0; e < 8; e++) sc.v[e] = widest[e] > 0.0f ? __fdiv_rn(widest[e], 255.0f) : 0.0f;
    }
    if (PASS == 1) st8(a + at, lo);
    if (PASS == 2) st8(b + at, sc);
}

// Values: LPR = D / 8 lanes per token, 64 / LPR tokens per wave.
template <typename SrcT, int BITS, int LPR>
__global__ void __launch_bounds__(256) kivi_quant_tokens_vec_kernel(const SrcT *__restrict__ src, int64_t S, int64_t src_t0, int n,
                                                                    uint8_t *__restrict__ codes, int64_t cap_rows, int64_t row0,
                                                                    float *__restrict__ lo_out, float *__restrict__ scale_out) {
    constexpr int D = LPR * 8, TPW = 64 / LPR, RB = D * BITS / 8;
    constexpr float lv = (float)((1u << BITS) - 1u);
    const int bh = blockIdx.y, lane = threadIdx.x & 63, sub = lane % LPR;
    const int i = (blockIdx.x * 4 + (threadIdx.x >> 6)) * TPW + lane / LPR;
    if (i >= n) return;   // whole groups of LPR lanes leave together; the exchanges below stay inside a group
    const F8 x = ld8(src + ((int64_t)bh * S + src_t0 + i) * D + sub * 8);
    float lo = INFINITY, hi = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        lo = fminf(lo, quiet(x.v[e]));
        hi = fmaxf(hi, quiet(x.v[e]));
    }
    group_min_max<LPR>(lo, hi);
    const float scale = affine_scale(lo, hi, lv), inv = affine_inv(scale);
    uint8_t *out_row = codes + ((int64_t)bh * cap_rows + row0 + i) * RB;
    if constexpr (BITS == 8) {
        uint32_t w0, w1;
        affine_words8_u8(x.v, lo, scale, inv, w0, w1);
        *reinterpret_cast<uint2 *>(out_row + sub * 8) = make_uint2(w0, w1);
    } else {
        uint32_t code[8];
        affine_codes8(x.v, lo, scale, inv, lv, code);
        store_codes8<BITS>(out_row, sub, code);
    }
    if (sub == 0) {
        lo_out[(int64_t)bh * cap_rows + row0 + i] = lo;
        scale_out[(int64_t)bh * cap_rows + row0 + i] = scale;
    }
}

// One decode step of QuantizedKvSdpa in one launch (head_dim 128, u8 codes): the new token's Key row into the running
// per-channel store (a thread per channel, as kivi_running_push_kernel) and its Value row into the per-token store (16
// lanes of 8 channels, as kivi_quant_tokens_vec_kernel).  Grid (batch * heads, 2) x 128 threads; sources [BH, 1, 128].
template <typename SrcT>
__global__ void __launch_bounds__(128) kivi_step_push_kernel(const SrcT *__restrict__ k_src, const SrcT *__restrict__ v_src,
                                                             uint8_t *__restrict__ k_codes, int64_t k_cap_rows, int64_t k_row0,
                                                             float *__restrict__ k_lo_io, float *__restrict__ k_scale_io,
                                                             uint8_t *__restrict__ v_codes, int64_t v_cap_rows, int64_t v_row0,
                                                             float *__restrict__ v_lo_out, float *__restrict__ v_scale_out) {
    constexpr int D = 128;
    const int bh = blockIdx.x;
    if (blockIdx.y == 0) {
        const int c = threadIdx.x;
        float lo = k_lo_io[(int64_t)bh * D + c], scale = k_scale_io[(int64_t)bh * D + c];
        const float val = ld(k_src + (int64_t)bh * D + c);
        if (val < lo) lo = val;
        const float range = __fsub_rn(val, lo);
        if (range > 0.0f) {
            const float ns = __fdiv_rn(range, 255.0f);
            if (ns > scale) scale = ns;
        }
        k_codes[((int64_t)bh * k_cap_rows + k_row0) * D + c] = (uint8_t)affine_code(val, lo, scale, 255.0f);
        k_lo_io[(int64_t)bh * D + c] = lo;
        k_scale_io[(int64_t)bh * D + c] = scale;
    } else {
        const int sub = threadIdx.x;
        if (sub >= 16) return;   // (the exchanges below stay inside the first 16 lanes)
        const F8 x = ld8(v_src + (int64_t)bh * D + sub * 8);
        float lo = INFINITY, hi = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            lo = fminf(lo, quiet(x.v[e]));
            hi = fmaxf(hi, quiet(x.v[e]));
        }
        group_min_max<16>(lo, hi);
        const float scale = affine_scale(lo, hi, 255.0f), inv = affine_inv(scale);
        uint32_t w0, w1;
        affine_words8_u8(x.v, lo, scale, inv, w0, w1);
        *reinterpret_cast<uint2 *>(v_codes + ((int64_t)bh * v_cap_rows + v_row0) * D + sub * 8) = make_uint2(w0, w1);
        if (sub == 0) {
            v_lo_out[(int64_t)bh * v_cap_rows + v_row0] = lo;
            v_scale_out[(int64_t)bh * v_cap_rows + v_row0] = scale;
        }
    }
}

// Keys: one wave per block whose 32 rows all come from the new tokens; the wave's 64 / LPR lane groups take the rows
// in turn, join their lo / hi, and code their rows in a second pass (the rows are in the cache by then).
template <typename SrcT, int BITS, int LPR>
__global__ void __launch_bounds__(256) kivi_finalize_blocks_vec_kernel(const SrcT *__restrict__ src, int64_t S, int64_t src_t0, int nb,
                                                                       const float *__restrict__ residual, int n_res_old,
                                                                       uint8_t *__restrict__ codes, int64_t cap_rows, int64_t row0,
                                                                       float *__restrict__ lo_out, float *__restrict__ scale_out) {
    constexpr int D = LPR * 8, G = 64 / LPR, RB = D * BITS / 8;
    constexpr float lv = (float)((1u << BITS) - 1u);
    const int bh = blockIdx.y, lane = threadIdx.x & 63, sub = lane % LPR, g = lane / LPR;
    const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (j >= nb) return;   // wave-uniform
    // row r of block j is row k = 32 j + r of the run: from the partial block when k < n_res_old, else new token k - n_res_old
    const SrcT *rows = src + ((int64_t)bh * S + src_t0 + (int64_t)j * kKeyBlock - n_res_old) * D + sub * 8;
    const float *res = residual + (int64_t)bh * kKeyBlock * D + sub * 8;
    const int n_old = j == 0 ? n_res_old : 0;
    float lo[8], hi[8], scale[8], inv[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        lo[e] = INFINITY;
        hi[e] = -INFINITY;
    }
    // (head sizes up to 128: a lane group's 4 or 8 rows stay in registers for the second pass)
    constexpr int RPG = kKeyBlock / G;          // rows per lane group
    constexpr bool KEEP = RPG <= 8;
    F8 keep[KEEP ? RPG : 1];
#pragma unroll (KEEP ? RPG : 4)
    for (int it = 0; it < RPG; it++) {   // row r = g + it G
        const int r = g + it * G;
        const F8 x = r < n_old ? ld8(res + (int64_t)r * D) : ld8(rows + (int64_t)r * D);
        if constexpr (KEEP) keep[it] = x;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            lo[e] = fminf(lo[e], quiet(x.v[e]));
            hi[e] = fmaxf(hi[e], quiet(x.v[e]));
        }
    }
    {   // the lane groups' rows joined: lanes LPR, 2 LPR, ... apart hold the same channels
        auto mn = [](float a, float b) { return fminf(a, b); };
        auto mx = [](float a, float b) { return fmaxf(a, b); };
#pragma unroll
        for (int e = 0; e < 8; e++) {
            if constexpr (LPR <= 8) lo[e] = xor_combine<8>(lo[e], mn), hi[e] = xor_combine<8>(hi[e], mx);
            if constexpr (LPR <= 16) lo[e] = xor_combine<16>(lo[e], mn), hi[e] = xor_combine<16>(hi[e], mx);
            if constexpr (LPR <= 32) lo[e] = xor_combine<32>(lo[e], mn), hi[e] = xor_combine<32>(hi[e], mx);
        }
    }
    F8 ls, ss;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        scale[e] = affine_scale(lo[e], hi[e], lv);
        inv[e] = affine_inv(scale[e]);
        ls.v[e] = lo[e];
        ss.v[e] = scale[e];
    }
    if (g == 0) {
        const int64_t at = ((int64_t)bh * (cap_rows / kKeyBlock) + row0 / kKeyBlock + j) * D + sub * 8;
        st8(lo_out + at, ls);
        st8(scale_out + at, ss);
    }
    uint8_t *out = codes + ((int64_t)bh * cap_rows + row0 + (int64_t)j * kKeyBlock) * RB;
#pragma unroll (KEEP ? RPG : 4)
    for (int it = 0; it < RPG; it++) {
        const int r = g + it * G;
        F8 x;
        if constexpr (KEEP) x = keep[it];
        else x = r < n_old ? ld8(res + (int64_t)r * D) : ld8(rows + (int64_t)r * D);
        if constexpr (BITS == 8) {
            uint32_t w0, w1;
            affine_words8_u8(x.v, lo, scale, inv, w0, w1);
            *reinterpret_cast<uint2 *>(out + (int64_t)r * RB + sub * 8) = make_uint2(w0, w1);
        } else {
            uint32_t code[8];
            affine_codes8(x.v, lo, scale, inv, lv, code);
            store_codes8<BITS>(out + (int64_t)r * RB, sub, code);
        }
    }
}

struct KiviView {
    int layout, D, row_bytes, len, n_sink, n_rows;
    int64_t sink_tokens, cap_rows;
    const float *sink, *residual, *lo, *scale;
    const uint8_t *codes;
};

// dequant_all (quant_dyn_kv_cache.rs:132-150, :200-229; kv_quant.rs:148-159, :224-234): dst [BH, len, D] dense.
template <typename DstT, int BITS>
__global__ void kivi_dequant_kernel(KiviView a, DstT *__restrict__ dst) {
    const int bh = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= a.len * a.D) return;
    const int t = e / a.D, c = e - t * a.D;
    float x;
    if (t < a.n_sink) {
        x = a.sink[((int64_t)bh * a.sink_tokens + t) * a.D + c];
    } else if (t - a.n_sink < a.n_rows) {
        const int r = t - a.n_sink;
        const uint8_t *row = a.codes + ((int64_t)bh * a.cap_rows + r) * a.row_bytes;
        uint32_t code;
        if (BITS == 8) {
            code = row[c];
        } else {
            const uint32_t b = row[c >> 1];
            code = (c & 1) ? (b >> 4) : (b & 15u);
        }
        int64_t p;
        if (a.layout == TROCM_KIVI_PER_TOKEN) p = (int64_t)bh * a.cap_rows + r;
        else if (a.layout == TROCM_KIVI_BLOCK_CHANNEL) p = ((int64_t)bh * (a.cap_rows / kKeyBlock) + r / kKeyBlock) * a.D + c;
        else p = (int64_t)bh * a.D + c;
        x = __fadd_rn(a.lo[p], __fmul_rn((float)code, a.scale[p]));
    } else {
        x = a.residual[((int64_t)bh * kKeyBlock + (t - a.n_sink - a.n_rows)) * a.D + c];
    }
    st(dst + ((int64_t)bh * a.len + t) * a.D + c, x);
}

// dequant_all for head sizes that are a multiple of 8: a thread owns 8 consecutive channels of one token.
// STREAM: the output leaves with streaming stores (the op's output, read much later); without it the stores stay in the
// caches for the attention launch that follows inside trocm_quantized_kv_sdpa_eval.
template <typename DstT, int BITS, bool STREAM>
__global__ void __launch_bounds__(256) kivi_dequant_vec_kernel(KiviView a, DstT *__restrict__ dst) {
    const int bh = blockIdx.y;
    const int d8 = a.D >> 3;
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < a.len * d8; e += gridDim.x * blockDim.x) {
    const int t = e / d8, c = (e - t * d8) * 8;
    F8 x;
    if (t < a.n_sink) {
        x = ld8(a.sink + ((int64_t)bh * a.sink_tokens + t) * a.D + c);
    } else if (t - a.n_sink < a.n_rows) {
        const int r = t - a.n_sink;
        const uint8_t *row = a.codes + ((int64_t)bh * a.cap_rows + r) * a.row_bytes;
        uint32_t code[8];
        if (BITS == 8) {
            const uint64_t w = __builtin_nontemporal_load(reinterpret_cast<const uint64_t *>(row + c));
#pragma unroll
            for (int i = 0; i < 8; i++) code[i] = (uint32_t)(w >> (8 * i)) & 255u;
        } else {
            const uint32_t w = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(row + (c >> 1)));
#pragma unroll
            for (int i = 0; i < 8; i++) code[i] = (w >> (4 * i)) & 15u;
        }
        if (a.layout == TROCM_KIVI_PER_TOKEN) {
            const float lo = a.lo[(int64_t)bh * a.cap_rows + r], sc = a.scale[(int64_t)bh * a.cap_rows + r];
#pragma unroll
            for (int i = 0; i < 8; i++) x.v[i] = __fadd_rn(lo, __fmul_rn((float)code[i], sc));
        } else {
            const int64_t p = a.layout == TROCM_KIVI_BLOCK_CHANNEL ? ((int64_t)bh * (a.cap_rows / kKeyBlock) + r / kKeyBlock) * a.D + c
                                                                   : (int64_t)bh * a.D + c;
            const F8 lo = ld8(a.lo + p), sc = ld8(a.scale + p);
#pragma unroll
            for (int i = 0; i < 8; i++) x.v[i] = __fadd_rn(lo.v[i], __fmul_rn((float)code[i], sc.v[i]));
        }
    } else {
        x = ld8(a.residual + ((int64_t)bh * kKeyBlock + (t - a.n_sink - a.n_rows)) * a.D + c);
    }
    if (STREAM) st8_stream(dst + ((int64_t)bh * a.len + t) * a.D + c, x);
    else st8(dst + ((int64_t)bh * a.len + t) * a.D + c, x);
    }
}

__global__ void kivi_fill_running_kernel(float *lo, float *scale, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        lo[i] = INFINITY;    // kv_quant.rs:187-188
        scale[i] = 1.0f;
    }
}

}  // namespace
}  // namespace trocm

using namespace trocm;

struct trocm_kivi_cache {
    int layout = 0, bits = 8;
    int64_t sink_tokens = 0, B = 0, H = 0, D = 0, BH = 0, row_bytes = 0;
    int64_t len = 0, n_sink = 0, n_rows = 0, n_res = 0, cap_rows = 0;
    float *sink = nullptr, *residual = nullptr, *lo = nullptr, *scale = nullptr;
    uint8_t *codes = nullptr;
    void *deq = nullptr;      // dequantised copy handed to attention by trocm_quantized_kv_sdpa_eval
    size_t deq_bytes = 0;
    float *scan = nullptr;    // chunk results of a prompt pushed into the running Key store (kept for the next prompt)
    size_t scan_bytes = 0;
};

static int64_t param_pitch(const trocm_kivi_cache *c, int64_t cap_rows) {
    switch (c->layout) {
        case TROCM_KIVI_PER_TOKEN: return cap_rows;
        case TROCM_KIVI_BLOCK_CHANNEL: return cap_rows / kKeyBlock * c->D;
        default: return c->D;
    }
}
static int64_t n_params(const trocm_kivi_cache *c) {
    switch (c->layout) {
        case TROCM_KIVI_PER_TOKEN: return c->n_rows;
        case TROCM_KIVI_BLOCK_CHANNEL: return c->n_rows / kKeyBlock * c->D;
        default: return c->D;
    }
}

// [BH rows of width_bytes] between two pitched planes.
static int copy_rows(void *dst, int64_t dpitch, const void *src, int64_t spitch, int64_t width, int64_t rows, hipStream_t s) {
    if (width == 0 || rows == 0) return 0;
    CopyNd d;
    d.rank = 2;
    d.shape[0] = rows;
    d.shape[1] = width;
    d.dst_stride[0] = dpitch;
    d.dst_stride[1] = 1;
    d.src_stride[0] = spitch;
    d.src_stride[1] = 1;
    return launch_copy_nd(dst, src, d, 1, s);
}

// hipMalloc that first gives memory waiting for its event a chance, and leaves no stale error behind when it fails (the
// next launch check would report it).
static int kivi_malloc(void **ptr, size_t bytes, const char *what) {
    *ptr = nullptr;
    hipError_t e = hipMalloc(ptr, bytes ? bytes : 16);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        reap_device_frees(true);
        e = hipMalloc(ptr, bytes ? bytes : 16);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *ptr = nullptr;
        return fail("allocating %s (%zu bytes) failed: %s", what, bytes, hipGetErrorString(e));
    }
    return 0;
}

static int kivi_alloc_fixed(trocm_kivi_cache *c, hipStream_t s) {
    if (c->sink_tokens && !c->sink && kivi_malloc((void **)&c->sink, (size_t)c->BH * c->sink_tokens * c->D * 4, "the unquantised first tokens")) return 1;
    if (c->layout == TROCM_KIVI_BLOCK_CHANNEL && !c->residual &&
        kivi_malloc((void **)&c->residual, (size_t)c->BH * kKeyBlock * c->D * 4, "the partial key block"))
        return 1;
    if (c->layout == TROCM_KIVI_RUNNING_CHANNEL && !c->lo) {
        const int64_t n = c->BH * c->D;
        float *lo = nullptr, *scale = nullptr;
        if (kivi_malloc((void **)&lo, (size_t)n * 4, "running key parameters")) return 1;
        if (kivi_malloc((void **)&scale, (size_t)n * 4, "running key parameters")) {
            (void)hipFree(lo);
            return 1;
        }
        c->lo = lo, c->scale = scale;
        kivi_fill_running_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, s>>>(c->lo, c->scale, n);
        TROCM_HIP(hipGetLastError());
    }
    return 0;
}

// Room for `need` coded rows: capacities are multiples of 32 and at least double.  The valid region moves on the
// stream; the old planes are released behind an event by a later call (the host does not wait for the stream).
static int kivi_ensure_rows(trocm_kivi_cache *c, int64_t need, hipStream_t s) {
    if (need <= c->cap_rows) return 0;
    int64_t cap = c->cap_rows * 2 > need ? c->cap_rows * 2 : need;
    cap = (cap + kKeyBlock - 1) / kKeyBlock * kKeyBlock;
    uint8_t *codes = nullptr;
    float *lo = nullptr, *scale = nullptr;
    if (kivi_malloc((void **)&codes, (size_t)c->BH * cap * c->row_bytes, "the codes of a quantised store")) return 1;
    const bool own_params = c->layout != TROCM_KIVI_RUNNING_CHANNEL;
    if (own_params) {
        if (kivi_malloc((void **)&lo, (size_t)c->BH * param_pitch(c, cap) * 4, "the parameters of a quantised store") ||
            kivi_malloc((void **)&scale, (size_t)c->BH * param_pitch(c, cap) * 4, "the parameters of a quantised store")) {
            (void)hipFree(codes);
            if (lo) (void)hipFree(lo);
            return 1;
        }
    }
    int rc = 0;
    if (c->n_rows) {
        rc = copy_rows(codes, cap * c->row_bytes, c->codes, c->cap_rows * c->row_bytes, c->n_rows * c->row_bytes, c->BH, s);
        if (!rc && own_params) {
            rc = copy_rows(lo, param_pitch(c, cap) * 4, c->lo, param_pitch(c, c->cap_rows) * 4, n_params(c) * 4, c->BH, s);
            if (!rc) rc = copy_rows(scale, param_pitch(c, cap) * 4, c->scale, param_pitch(c, c->cap_rows) * 4, n_params(c) * 4, c->BH, s);
        }
    }
    if (rc) {
        (void)hipFree(codes);
        if (lo) (void)hipFree(lo);
        if (scale) (void)hipFree(scale);
        return rc;
    }
    if (c->codes) {   // the copies above (and whatever the stream still runs over the old planes) finish first
        if (defer_device_free(c->codes, nullptr, s)) return 1;
        if (own_params && defer_device_free(c->lo, c->scale, s)) return 1;
    }
    c->codes = codes;
    if (own_params) {
        c->lo = lo;
        c->scale = scale;
    }
    c->cap_rows = cap;
    return 0;
}

// A scratch buffer that only grows (by doubling); the one it replaces is released behind an event.
static int kivi_grow_buffer(void **buf, size_t *have, size_t need, hipStream_t s, const char *what) {
    if (*have >= need) return 0;
    const size_t cap = *have * 2 > need ? *have * 2 : need;
    void *fresh = nullptr;
    if (kivi_malloc(&fresh, cap, what)) return 1;
    if (*buf && defer_device_free(*buf, nullptr, s)) return 1;
    *buf = fresh;
    *have = cap;
    return 0;
}

static bool kivi_prompt_scan(const trocm_kivi_cache *c, int64_t rem) {
    return c->layout == TROCM_KIVI_RUNNING_CHANNEL && rem >= 4 * kRunChunk && (rem + kRunChunk - 1) / kRunChunk <= 65535;
}

// Everything an append of S tokens may have to allocate, before anything is launched or counted: a call that fails here
// has changed nothing and can be repeated.
static int kivi_prepare(trocm_kivi_cache *c, int64_t S, hipStream_t s) {
    if (kivi_alloc_fixed(c, s)) return 1;
    const int64_t ns = c->sink_tokens - c->n_sink < S ? c->sink_tokens - c->n_sink : S;
    const int64_t rem = S - (ns > 0 ? ns : 0);
    if (rem <= 0) return 0;
    int64_t rows = c->n_rows + rem;
    if (c->layout == TROCM_KIVI_BLOCK_CHANNEL) rows = c->n_rows + (c->n_res + rem) / kKeyBlock * kKeyBlock;
    if (rows > c->n_rows && kivi_ensure_rows(c, rows, s)) return 1;
    if (kivi_prompt_scan(c, rem)) {
        const size_t need = (size_t)c->BH * ((rem + kRunChunk - 1) / kRunChunk) * c->D * 3 * sizeof(float);   // (three results per chunk and channel on the 128-bit path)
        if (kivi_grow_buffer((void **)&c->scan, &c->scan_bytes, need, s, "the chunk results of a prompt")) return 1;
    }
    return 0;
}

template <typename SrcT>
static int kivi_append_t(trocm_kivi_cache *c, const SrcT *src, int64_t S, hipStream_t s) {
    const int D = (int)c->D;
    const unsigned BH = (unsigned)c->BH;
    if (kivi_prepare(c, S, s)) return 1;   // every allocation of this call: nothing below can run out of memory
    int64_t t0 = 0;
    const int64_t ns = c->sink_tokens - c->n_sink < S ? c->sink_tokens - c->n_sink : S;
    if (ns > 0) {   // quant_dyn_kv_cache.rs:118-122, :170-174
        kivi_rows_to_f32_kernel<SrcT><<<dim3((unsigned)((ns * D + 255) / 256), BH), 256, 0, s>>>(src, S, 0, c->sink, c->sink_tokens, c->n_sink, (int)ns, D);
        TROCM_HIP(hipGetLastError());
        c->n_sink += ns;
        t0 = ns;
    }
    const int64_t rem = S - t0;
    if (rem > 0 && c->layout == TROCM_KIVI_PER_TOKEN) {
        const bool vec = ((uintptr_t)src & 15) == 0 && (D == 64 || D == 128 || D == 256 || D == 512);
#define KIVI_TOKENS_VEC(BITS, LPR)                                                                                              \
    kivi_quant_tokens_vec_kernel<SrcT, BITS, LPR><<<dim3((unsigned)((rem + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))), BH), 256, 0, s>>>( \
        src, S, t0, (int)rem, c->codes, c->cap_rows, c->n_rows, c->lo, c->scale)
        if (vec && c->bits == 8) {
            if (D == 64) KIVI_TOKENS_VEC(8, 8); else if (D == 128) KIVI_TOKENS_VEC(8, 16); else if (D == 256) KIVI_TOKENS_VEC(8, 32); else KIVI_TOKENS_VEC(8, 64);
        } else if (vec) {
            if (D == 64) KIVI_TOKENS_VEC(4, 8); else if (D == 128) KIVI_TOKENS_VEC(4, 16); else if (D == 256) KIVI_TOKENS_VEC(4, 32); else KIVI_TOKENS_VEC(4, 64);
        } else {
            const dim3 grid((unsigned)((rem + 3) / 4), BH);
            if (c->bits == 8)
                kivi_quant_tokens_kernel<SrcT, 8><<<grid, 256, 0, s>>>(src, S, t0, (int)rem, D, c->codes, c->cap_rows, (int)c->row_bytes, c->n_rows, c->lo, c->scale);
            else
                kivi_quant_tokens_kernel<SrcT, 4><<<grid, 256, 0, s>>>(src, S, t0, (int)rem, D, c->codes, c->cap_rows, (int)c->row_bytes, c->n_rows, c->lo, c->scale);
        }
#undef KIVI_TOKENS_VEC
        TROCM_HIP(hipGetLastError());
        c->n_rows += rem;
    } else if (rem > 0 && c->layout == TROCM_KIVI_BLOCK_CHANNEL) {
        const int64_t nb = (c->n_res + rem) / kKeyBlock;
        if (nb > 0) {
            const bool vec = ((uintptr_t)src & 15) == 0 && (D == 64 || D == 128 || D == 256 || D == 512);
#define KIVI_BLOCKS_VEC(BITS, LPR)                                                                               \
    kivi_finalize_blocks_vec_kernel<SrcT, BITS, LPR><<<dim3((unsigned)((nb + 3) / 4), BH), 256, 0, s>>>(         \
        src, S, t0, (int)nb, c->residual, (int)c->n_res, c->codes, c->cap_rows, c->n_rows, c->lo, c->scale)
            if (vec && c->bits == 8) {
                if (D == 64) KIVI_BLOCKS_VEC(8, 8); else if (D == 128) KIVI_BLOCKS_VEC(8, 16); else if (D == 256) KIVI_BLOCKS_VEC(8, 32); else KIVI_BLOCKS_VEC(8, 64);
            } else if (vec) {
                if (D == 64) KIVI_BLOCKS_VEC(4, 8); else if (D == 128) KIVI_BLOCKS_VEC(4, 16); else if (D == 256) KIVI_BLOCKS_VEC(4, 32); else KIVI_BLOCKS_VEC(4, 64);
            } else {
                const dim3 grid((unsigned)nb, BH);
                const int threads = c->row_bytes >= 256 ? 256 : (int)((c->row_bytes + 63) / 64 * 64);
                if (c->bits == 8)
                    kivi_finalize_blocks_kernel<SrcT, 8><<<grid, threads, 0, s>>>(src, S, t0, c->residual, (int)c->n_res, D, c->codes, c->cap_rows, (int)c->row_bytes, c->n_rows, c->lo, c->scale);
                else
                    kivi_finalize_blocks_kernel<SrcT, 4><<<grid, threads, 0, s>>>(src, S, t0, c->residual, (int)c->n_res, D, c->codes, c->cap_rows, (int)c->row_bytes, c->n_rows, c->lo, c->scale);
            }
#undef KIVI_BLOCKS_VEC
            TROCM_HIP(hipGetLastError());
            const int64_t used = nb * kKeyBlock - c->n_res, tail = rem - used;
            c->n_rows += nb * kKeyBlock;
            if (tail > 0) {
                kivi_rows_to_f32_kernel<SrcT><<<dim3((unsigned)((tail * D + 255) / 256), BH), 256, 0, s>>>(src, S, t0 + used, c->residual, kKeyBlock, 0, (int)tail, D);
                TROCM_HIP(hipGetLastError());
            }
            c->n_res = tail;
        } else {
            kivi_rows_to_f32_kernel<SrcT><<<dim3((unsigned)((rem * D + 255) / 256), BH), 256, 0, s>>>(src, S, t0, c->residual, kKeyBlock, c->n_res, (int)rem, D);
            TROCM_HIP(hipGetLastError());
            c->n_res += rem;
        }
    } else if (rem > 0) {
        const int64_t n_chunks = (rem + kRunChunk - 1) / kRunChunk;
        if (kivi_prompt_scan(c, rem)) {   // a prompt: chunks side by side (scratch: two floats per chunk and channel)
            float *tmp = c->scan;
            const size_t plane = (size_t)c->BH * n_chunks * D;
            const SrcT *from = src + t0 * D;
            const dim3 scan((unsigned)((D + 63) / 64), BH);
            const bool vec = ((uintptr_t)from & 15) == 0 && (D == 64 || D == 128 || D == 256 || D == 512);
#define KIVI_RUN_VEC(LPR)                                                                                                              \
    do {                                                                                                                               \
        const dim3 vgrid((unsigned)((n_chunks + 256 / LPR - 1) / (256 / LPR)), BH);                                                    \
        kivi_run_chunk_vec_kernel<SrcT, LPR, 12><<<vgrid, 256, 0, s>>>(from, S, (int)rem, (int)n_chunks, tmp, tmp + plane, c->codes, c->cap_rows, c->n_rows, tmp + 2 * plane); \
        kivi_run_scan_both_kernel<<<scan, 64, 0, s>>>(tmp, tmp + plane, tmp + 2 * plane, D, (int)n_chunks, c->lo, c->scale);         \
        kivi_run_chunk_vec_kernel<SrcT, LPR, 3><<<vgrid, 256, 0, s>>>(from, S, (int)rem, (int)n_chunks, tmp, tmp + plane, c->codes, c->cap_rows, c->n_rows); \
    } while (0)
            if (vec) {
                if (D == 64) KIVI_RUN_VEC(8); else if (D == 128) KIVI_RUN_VEC(16); else if (D == 256) KIVI_RUN_VEC(32); else KIVI_RUN_VEC(64);
            } else {
                const dim3 grid((unsigned)((D + 63) / 64), (unsigned)n_chunks, BH);
                kivi_run_chunk_min_kernel<SrcT><<<grid, 64, 0, s>>>(from, S, (int)rem, D, (int)n_chunks, tmp);
                kivi_run_scan_min_kernel<<<scan, 64, 0, s>>>(tmp, D, (int)n_chunks, c->lo);
                kivi_run_chunk_scale_kernel<SrcT><<<grid, 64, 0, s>>>(from, S, (int)rem, D, (int)n_chunks, tmp, tmp + plane);
                kivi_run_scan_scale_kernel<<<scan, 64, 0, s>>>(tmp + plane, D, (int)n_chunks, c->scale);
                kivi_run_chunk_codes_kernel<SrcT><<<grid, 64, 0, s>>>(from, S, (int)rem, D, (int)n_chunks, tmp, tmp + plane, c->codes, c->cap_rows, c->n_rows);
            }
#undef KIVI_RUN_VEC
            TROCM_HIP(hipGetLastError());
        } else {
            kivi_running_push_kernel<SrcT><<<dim3((unsigned)((D + 127) / 128), BH), 128, 0, s>>>(src + t0 * D, S, (int)rem, D, c->codes, c->cap_rows, c->n_rows, c->lo, c->scale);
            TROCM_HIP(hipGetLastError());
        }
        c->n_rows += rem;
    }
    c->len += S;
    return 0;
}

static int kivi_dequantize(const trocm_kivi_cache *c, void *dst, int dst_dtype, hipStream_t s, bool stream_out = true) {
    if (c->len == 0) return 0;
    KiviView a;
    a.layout = c->layout;
    a.D = (int)c->D;
    a.row_bytes = (int)c->row_bytes;
    a.len = (int)c->len;
    a.n_sink = (int)c->n_sink;
    a.n_rows = (int)c->n_rows;
    a.sink_tokens = c->sink_tokens;
    a.cap_rows = c->cap_rows;
    a.sink = c->sink;
    a.residual = c->residual;
    a.lo = c->lo;
    a.scale = c->scale;
    a.codes = c->codes;
    if (c->D % 8 == 0 && ((uintptr_t)dst & 15) == 0) {
        int64_t gx = (c->len * (c->D / 8) + 255) / 256;
        // at most 128 workgroups per compute unit, whose threads then take several trips (8 x 8 x 16384 x 128 to f16: one
        // trip per thread 84 us, 128 per compute unit 78, 64: 79, 32: 82, 16: 93)
        const int64_t want = (int64_t)num_compute_units() * 128;
        if (gx * c->BH > want) gx = (want + c->BH - 1) / c->BH;
        const dim3 grid8((unsigned)gx, (unsigned)c->BH);
#define KIVI_DEQ(T, BITS)                                                                          \
    do {                                                                                           \
        if (stream_out) kivi_dequant_vec_kernel<T, BITS, true><<<grid8, 256, 0, s>>>(a, (T *)dst); \
        else kivi_dequant_vec_kernel<T, BITS, false><<<grid8, 256, 0, s>>>(a, (T *)dst);          \
    } while (0)
        if (dst_dtype == TROCM_F32) {
            if (c->bits == 8) KIVI_DEQ(float, 8);
            else KIVI_DEQ(float, 4);
        } else {
            if (c->bits == 8) KIVI_DEQ(__half, 8);
            else KIVI_DEQ(__half, 4);
        }
#undef KIVI_DEQ
        TROCM_HIP(hipGetLastError());
        return 0;
    }
    const dim3 grid((unsigned)((c->len * c->D + 255) / 256), (unsigned)c->BH);
    if (dst_dtype == TROCM_F32) {
        if (c->bits == 8) kivi_dequant_kernel<float, 8><<<grid, 256, 0, s>>>(a, (float *)dst);
        else kivi_dequant_kernel<float, 4><<<grid, 256, 0, s>>>(a, (float *)dst);
    } else {
        if (c->bits == 8) kivi_dequant_kernel<__half, 8><<<grid, 256, 0, s>>>(a, (__half *)dst);
        else kivi_dequant_kernel<__half, 4><<<grid, 256, 0, s>>>(a, (__half *)dst);
    }
    TROCM_HIP(hipGetLastError());
    return 0;
}

extern "C" {

int trocm_kivi_cache_create(trocm_kivi_cache **out, int layout, int bits, int64_t sink_tokens, int64_t batch,
                            int64_t heads, int64_t head_dim) {
    TROCM_NOT_NULL(out);
    if (ensure_init()) return 1;
    TROCM_REQUIRE(layout == TROCM_KIVI_PER_TOKEN || layout == TROCM_KIVI_BLOCK_CHANNEL || layout == TROCM_KIVI_RUNNING_CHANNEL,
                  "unknown quantised-cache layout %d", layout);
    TROCM_REQUIRE(bits == 4 || bits == 8, "KV quantization bits must be 4 or 8");   // quant_dyn_kv_cache.rs:706
    TROCM_REQUIRE(layout != TROCM_KIVI_RUNNING_CHANNEL || bits == 8, "the running per-channel key store holds 8-bit codes");
    TROCM_REQUIRE(batch > 0 && heads > 0 && head_dim > 0 && sink_tokens >= 0, "quantised cache: invalid shape");
    TROCM_REQUIRE(batch * heads <= 65535, "quantised cache: batch * heads = %lld exceeds 65535", (long long)(batch * heads));
    trocm_kivi_cache *c = new (std::nothrow) trocm_kivi_cache();
    TROCM_REQUIRE(c, "out of host memory");
    c->layout = layout;
    c->bits = bits;
    c->sink_tokens = sink_tokens;
    c->B = batch;
    c->H = heads;
    c->D = head_dim;
    c->BH = batch * heads;
    c->row_bytes = (head_dim * bits + 7) / 8;   // quant_dyn_kv_cache.rs:58-60
    *out = c;
    return 0;
}

int trocm_kivi_cache_destroy(trocm_kivi_cache *c) {
    if (!c) return 0;
    (void)hipFree(c->sink);
    (void)hipFree(c->residual);
    (void)hipFree(c->lo);
    (void)hipFree(c->scale);
    (void)hipFree(c->codes);
    (void)hipFree(c->deq);
    (void)hipFree(c->scan);
    delete c;
    return 0;
}

int trocm_kivi_cache_reset(trocm_kivi_cache *c, void *stream) {
    TROCM_NOT_NULL(c);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    c->len = c->n_sink = c->n_rows = c->n_res = 0;
    if (c->layout == TROCM_KIVI_RUNNING_CHANNEL && c->lo) {
        const int64_t n = c->BH * c->D;
        kivi_fill_running_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, s>>>(c->lo, c->scale, n);
        TROCM_HIP(hipGetLastError());
    }
    return 0;
}

int trocm_kivi_cache_len(const trocm_kivi_cache *c, int64_t *len) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(len);
    *len = c->len;
    return 0;
}

int trocm_kivi_cache_counts(const trocm_kivi_cache *c, int64_t *n_sink, int64_t *n_rows, int64_t *n_res, int64_t *row_bytes) {
    TROCM_NOT_NULL(c);
    if (n_sink) *n_sink = c->n_sink;
    if (n_rows) *n_rows = c->n_rows;
    if (n_res) *n_res = c->n_res;
    if (row_bytes) *row_bytes = c->row_bytes;
    return 0;
}

int trocm_kivi_cache_memory_bytes(const trocm_kivi_cache *c, size_t *bytes) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(bytes);
    const size_t per_head = (size_t)(c->n_rows * c->row_bytes) + (size_t)n_params(c) * 8 + (size_t)(c->n_sink + c->n_res) * c->D * 4;
    *bytes = per_head * (size_t)c->BH;
    return 0;
}

int trocm_kivi_cache_append(trocm_kivi_cache *c, const void *src, int src_dtype, int64_t n_new, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(src_dtype == TROCM_F32 || src_dtype == TROCM_F16, "quantised cache: the input must be f32 or f16");
    TROCM_REQUIRE(n_new >= 0, "quantised cache: negative token count");
    if (n_new == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_REQUIRE((c->len + n_new) * c->D < (1ll << 31) && n_new * c->D < (1ll << 31), "quantised cache: %lld tokens of %lld channels exceed the index range",
                  (long long)(c->len + n_new), (long long)c->D);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return src_dtype == TROCM_F32 ? kivi_append_t(c, (const float *)src, n_new, s) : kivi_append_t(c, (const __half *)src, n_new, s);
}

int trocm_kivi_cache_dequantize(const trocm_kivi_cache *c, void *dst, int dst_dtype, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(dst_dtype == TROCM_F32 || dst_dtype == TROCM_F16, "quantised cache: the output must be f32 or f16");
    if (c->len == 0) return 0;
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return kivi_dequantize(c, dst, dst_dtype, s);
}

int trocm_kivi_cache_export(const trocm_kivi_cache *c, int part, void *dst, size_t *bytes, void *stream) {
    TROCM_NOT_NULL(c);
    int64_t width = 0, pitch = 0;
    const void *src = nullptr;
    switch (part) {
        case TROCM_KIVI_PART_SINK: width = c->n_sink * c->D * 4; pitch = c->sink_tokens * c->D * 4; src = c->sink; break;
        case TROCM_KIVI_PART_CODES: width = c->n_rows * c->row_bytes; pitch = c->cap_rows * c->row_bytes; src = c->codes; break;
        case TROCM_KIVI_PART_LO: width = n_params(c) * 4; pitch = param_pitch(c, c->cap_rows) * 4; src = c->lo; break;
        case TROCM_KIVI_PART_SCALE: width = n_params(c) * 4; pitch = param_pitch(c, c->cap_rows) * 4; src = c->scale; break;
        case TROCM_KIVI_PART_RESIDUAL: width = c->n_res * c->D * 4; pitch = (int64_t)kKeyBlock * c->D * 4; src = c->residual; break;
        default: return fail("quantised cache: unknown part %d", part);
    }
    if (c->layout == TROCM_KIVI_RUNNING_CHANNEL && (part == TROCM_KIVI_PART_LO || part == TROCM_KIVI_PART_SCALE) && !c->lo) width = 0;
    if (bytes) *bytes = (size_t)width * (size_t)c->BH;
    if (!dst || width == 0) return 0;
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return copy_rows(dst, width, src, pitch, width, c->BH, s);
}

int trocm_kivi_cache_clone(const trocm_kivi_cache *c, trocm_kivi_cache **out, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(out);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    trocm_kivi_cache *n = nullptr;
    if (trocm_kivi_cache_create(&n, c->layout, c->bits, c->sink_tokens, c->B, c->H, c->D)) return 1;
    int rc = 0;
    if (c->len > 0) {
        rc = kivi_alloc_fixed(n, s);
        if (!rc && c->n_rows) rc = kivi_ensure_rows(n, c->cap_rows, s);
        n->len = c->len;
        n->n_sink = c->n_sink;
        n->n_rows = c->n_rows;
        n->n_res = c->n_res;
        if (!rc && c->n_sink) rc = copy_rows(n->sink, c->sink_tokens * c->D * 4, c->sink, c->sink_tokens * c->D * 4, c->n_sink * c->D * 4, c->BH, s);
        if (!rc && c->n_res) rc = copy_rows(n->residual, (int64_t)kKeyBlock * c->D * 4, c->residual, (int64_t)kKeyBlock * c->D * 4, c->n_res * c->D * 4, c->BH, s);
        if (!rc && c->n_rows) rc = copy_rows(n->codes, n->cap_rows * c->row_bytes, c->codes, c->cap_rows * c->row_bytes, c->n_rows * c->row_bytes, c->BH, s);
        if (!rc && c->lo && n_params(c)) {
            rc = copy_rows(n->lo, param_pitch(n, n->cap_rows) * 4, c->lo, param_pitch(c, c->cap_rows) * 4, n_params(c) * 4, c->BH, s);
            if (!rc) rc = copy_rows(n->scale, param_pitch(n, n->cap_rows) * 4, c->scale, param_pitch(c, c->cap_rows) * 4, n_params(c) * 4, c->BH, s);
        }
    }
    if (rc) {
        trocm_kivi_cache_destroy(n);
        return rc;
    }
    *out = n;
    return 0;
}

// One token of f16 queries over the op's own stores (Keys under running per-channel parameters, Values per token, u8
// codes, nothing kept in f32): attention straight over the codes, no dequantised copy.  TROCM_KIVI_FUSED=0 keeps the
// dequantising path, which serves every other case.  (Evaluated before the step's tokens are appended: the stores
// hold whole coded rows only, so the conditions on their counts hold afterwards as well.)
static bool kivi_fused_step(int dtype, int64_t n_new, const trocm_kivi_cache *k, const trocm_kivi_cache *v) {
    static const int fused = getenv("TROCM_KIVI_FUSED") ? atoi(getenv("TROCM_KIVI_FUSED")) : 1;
    return fused && dtype == TROCM_F16 && n_new == 1 && k->D == 128 && k->layout == TROCM_KIVI_RUNNING_CHANNEL &&
           v->layout == TROCM_KIVI_PER_TOKEN && k->bits == 8 && v->bits == 8 && k->sink_tokens == 0 && v->sink_tokens == 0 &&
           k->n_res == 0 && v->n_res == 0 && k->n_rows == k->len && v->n_rows == v->len;
}

int trocm_quantized_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                                 int64_t n_new, trocm_kivi_cache *k_cache, trocm_kivi_cache *v_cache, void *out,
                                 float scale, void *workspace, size_t workspace_bytes, void *stream) {
    TROCM_NOT_NULL(q);
    TROCM_NOT_NULL(k_new);
    TROCM_NOT_NULL(v_new);
    TROCM_NOT_NULL(k_cache);
    TROCM_NOT_NULL(v_cache);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE(dtype == TROCM_F32 || dtype == TROCM_F16, "QuantizedKvSdpa: inputs must be f32 or f16");
    TROCM_REQUIRE(n_new > 0, "QuantizedKvSdpa: no new token");
    TROCM_REQUIRE(k_cache->B == v_cache->B && k_cache->H == v_cache->H && k_cache->D == v_cache->D && k_cache->len == v_cache->len,
                  "QuantizedKvSdpa: the K and V stores differ in shape or length");
    TROCM_REQUIRE(q_heads > 0 && q_heads % k_cache->H == 0, "QuantizedKvSdpa: %lld query heads over %lld kv heads",
                  (long long)q_heads, (long long)k_cache->H);
    TROCM_REQUIRE((k_cache->len + n_new) * k_cache->D < (1ll << 31) && n_new * k_cache->D < (1ll << 31),
                  "QuantizedKvSdpa: %lld tokens of %lld channels exceed the index range", (long long)(k_cache->len + n_new), (long long)k_cache->D);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    // Every allocation of the step, for both stores, before either is touched: a call that fails for want of memory
    // leaves K and V as they were (same length, same counts) and can be repeated.
    const bool fused_attention = kivi_fused_step(dtype, n_new, k_cache, v_cache);
    for (trocm_kivi_cache *c : {k_cache, v_cache})
        if (kivi_prepare(c, n_new, s)) return 1;
    if (!(fused_attention && workspace)) {
        const size_t need = (size_t)k_cache->BH * (k_cache->len + n_new) * k_cache->D * elem_bytes(dtype);
        for (trocm_kivi_cache *c : {k_cache, v_cache})
            if (kivi_grow_buffer(&c->deq, &c->deq_bytes, need, s, "the dequantised copy of a quantised store")) return 1;
    }
    // a decode step on the op's own stores: both rows pushed by one launch
    if (n_new == 1 && k_cache->D == 128 && k_cache->layout == TROCM_KIVI_RUNNING_CHANNEL && v_cache->layout == TROCM_KIVI_PER_TOKEN &&
        k_cache->bits == 8 && v_cache->bits == 8 && k_cache->sink_tokens == 0 && v_cache->sink_tokens == 0 &&
        ((uintptr_t)v_new & 15) == 0 && (k_cache->len + 1) * 128 < (1ll << 31)) {
        const dim3 grid((unsigned)k_cache->BH, 2);
        if (dtype == TROCM_F16)
            kivi_step_push_kernel<__half><<<grid, 128, 0, s>>>((const __half *)k_new, (const __half *)v_new, k_cache->codes, k_cache->cap_rows, k_cache->n_rows,
                                                               k_cache->lo, k_cache->scale, v_cache->codes, v_cache->cap_rows, v_cache->n_rows, v_cache->lo, v_cache->scale);
        else
            kivi_step_push_kernel<float><<<grid, 128, 0, s>>>((const float *)k_new, (const float *)v_new, k_cache->codes, k_cache->cap_rows, k_cache->n_rows,
                                                              k_cache->lo, k_cache->scale, v_cache->codes, v_cache->cap_rows, v_cache->n_rows, v_cache->lo, v_cache->scale);
        TROCM_HIP(hipGetLastError());
        for (trocm_kivi_cache *c : {k_cache, v_cache}) c->n_rows += 1, c->len += 1;
    } else {
        if (trocm_kivi_cache_append(k_cache, k_new, dtype, n_new, s)) return 1;
        if (trocm_kivi_cache_append(v_cache, v_new, dtype, n_new, s)) return 1;
    }
    const int64_t T = k_cache->len, D = k_cache->D;
    // One token of f16 queries over the op's own stores (Keys under running per-channel parameters, Values per token, u8
    // codes, nothing kept in f32): attention straight over the codes, no dequantised copy.  TROCM_KIVI_FUSED=0 keeps
    // the dequantising path below, which serves every other case.
    if (fused_attention) {
        KiviSdpaArgs a;
        a.q = q, a.out = out;
        a.k_codes = k_cache->codes, a.v_codes = v_cache->codes;
        a.k_cap_rows = k_cache->cap_rows, a.v_cap_rows = v_cache->cap_rows;
        a.k_chan_scale = k_cache->scale;
        a.v_tok_scale = v_cache->scale, a.v_tok_lo = v_cache->lo;
        a.B = k_cache->B, a.Hq = q_heads, a.Hkv = k_cache->H, a.T = T;
        a.scale = scale == scale ? scale : 1.0f / sqrtf((float)D);   // NaN asks for the default (sdpa.rs:93-95)
        a.workspace = workspace, a.workspace_bytes = workspace_bytes;
        const int rc = workspace ? launch_sdpa_decode_kivi(a, s) : 2;
        if (rc == 0) {   // the dequantised copies a prompt left behind are not needed again: released behind an event
            for (trocm_kivi_cache *c : {k_cache, v_cache})
                if (c->deq) {
                    if (defer_device_free(c->deq, nullptr, s)) return 1;
                    c->deq = nullptr;
                    c->deq_bytes = 0;
                }
        }
        if (rc != 2) return rc;
        // (the launch declined: the dequantising path needs its buffers after all)
        const size_t need = (size_t)k_cache->BH * T * D * elem_bytes(dtype);
        for (trocm_kivi_cache *c : {k_cache, v_cache})
            if (kivi_grow_buffer(&c->deq, &c->deq_bytes, need, s, "the dequantised copy of a quantised store")) return 1;
    }
    for (trocm_kivi_cache *c : {k_cache, v_cache})
        if (kivi_dequantize(c, c->deq, dtype, s, false)) return 1;
    const int64_t strides[3] = {k_cache->H * T * D, T * D, D};
    // kv_quant.rs:326-327: FlashSdpaOp { causal: false, scale }
    return trocm_sdpa(q, k_cache->deq, v_cache->deq, nullptr, out, dtype, k_cache->B, q_heads, k_cache->H, n_new, T, D, strides, 1, 1,
                      scale, 0, workspace, workspace_bytes, s);
}

}  // extern "C"
