// Q4_0 weights x 2..16 f16 activation rows on the matrix cores: gfx950.
//
//   out[b, i, j] = sum_k act[b, i, k] * dequant(W[b / ratio, j, k]),   2 <= i-count m <= 16
//
// the rows of a batched decode step or of a short speculative run through GgmlGemm
// (cuda/src/kernels/matmul/mod.rs:575-627).  The vector-ALU kernel of q4_matvec.hip multiplies every
// weight by each of the m rows in turn (its time grows with m: 9.5 us for one row of a 14336 x 4096
// matrix, 39.5 us for eight); here one v_mfma_f32_16x16x32_f16 multiplies a block of 16 weight rows by up
// to 16 activation rows, so the launch stays bound by the weights' bytes.
//
// Arithmetic: the contraction of the instruction is 32 deep, exactly one quantisation block.  The codes enter
// as the exact f16 integers -8..7, the products accumulate in f32 inside the instruction from zero, and the
// block's sum is scaled by its f16 scale with one fma per output: the definition the vector-ALU kernel
// computes, in another order of additions.
//
// Work: KS waves (4, or 8 when the matrix has too few rows to occupy every SIMD otherwise) own 16 R weight rows; each
// walks one contiguous share of k, and they add their partial sums through LDS at the end.  A workgroup holds S
// such sets behind one staged chunk of the activations.  The instruction wants from lane (r, g) (r = l % 16,
// g = l / 16) byte group g of a block of weight row r, i.e. its codes 4g..4g+3 and 16+4g..16+4g+3.  The codes are
// loaded 128 contiguous bytes (8 blocks) of 8 rows per instruction and passed through 16 x 144 bytes of LDS of the
// wave's own, from which every lane reads its four bytes per instruction (a load instruction costs the compute
// unit's address path one step per cache line it touches, whatever it uses of the line); where LDS has no room for
// that, lane (r, g) loads the 16 bytes of block 4 i + g of row r and a 4 x 4 transpose over the lane groups
// (v_permlane32_swap, v_permlane16_swap) hands it byte group g of blocks 4 i .. 4 i + 3.  The activations are staged in LDS in that
// feature order (16-byte vectors XOR-swizzled by row, so that the 16 rows of one read fall into different
// banks) and read as the A operand.  When they do not fit, they are staged in chunks of 2048 features that hold a
// piece of every wave's share of k, so that a wave's weights stay one contiguous stream that is prefetched across
// the chunks, and the next chunk's activations wait in registers while this chunk is multiplied.
//
// Roofline: HBM-bound on the weights: 18 bytes per 32 weights, read once.
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// KS waves split the features of one set of 16 R rows (4, or 8 when the matrix has few rows); each keeps PD = 16 / KS
// groups of four blocks per row in flight ahead of the arithmetic.

struct MvMfmaDev {
    const uint8_t *codes;     // [w_batch, n, k/2]
    const uint16_t *scales;   // [w_batch, n, k/32]
    const _Float16 *act;      // [act_batch, m, k]
    _Float16 *out;            // [act_batch, m, n]
    int64_t act_stride_b, out_stride_b;   // elements between consecutive batches of act and out
    int n, k, m, ratio;       // ratio = act_batch / w_batch
    int cq;                   // groups of four blocks (128 features) per quarter of k in one staged chunk
    int nch;                  // chunks; 1 = the activations fit in LDS and are staged once per workgroup
    int prefetch;             // the next chunk's activations wait in registers during this chunk's arithmetic
    int wide;                 // 128-byte loads of 8 rows through the waves' code buffers (host-side choice of the kernel)
    int groups;               // row groups of 16 R S rows
};
constexpr int kCodeRow = 144;   // bytes between the rows of a wave's pair of code groups in LDS (128 + 16: no bank conflicts)
constexpr int kStageRegs = 8;   // 8-byte pieces of the next chunk a thread holds (prefetch mode)
// cq in prefetch mode is PD: a chunk is 2048 features, 512 pieces per row, and piece indices split by shifts

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// The four bytes of `c` hold codes (low nibbles) e..e+3 and (high nibbles) 16+e..16+e+3 of a block: the eight
// values code - 8 as f16, in that order.  0x6400 | v is the half 1024 + v; 1032 comes off exactly.
__device__ __forceinline__ half8_t codes_as_halves(uint32_t c) {
    const uint32_t lo = c & 0x0F0F0F0Fu, hi = (c >> 4) & 0x0F0F0F0Fu;
    const half2_t off = {(_Float16)1032.0f, (_Float16)1032.0f};
    const half2_t a = __builtin_bit_cast(half2_t, perm(0x64646464u, lo, 0x04010400u)) - off;
    const half2_t b = __builtin_bit_cast(half2_t, perm(0x64646464u, lo, 0x04030402u)) - off;
    const half2_t c2 = __builtin_bit_cast(half2_t, perm(0x64646464u, hi, 0x04010400u)) - off;
    const half2_t d = __builtin_bit_cast(half2_t, perm(0x64646464u, hi, 0x04030402u)) - off;
    return half8_t{a[0], a[1], b[0], b[1], c2[0], c2[1], d[0], d[1]};
}

// Register j of lane group g <-> register g of lane group j (lane groups of 16 lanes).
__device__ __forceinline__ void transpose_lane_groups(u32x4 &w) {
    auto s02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);   // upper half of [0] <-> lower half of [2]
    auto s13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
    auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);   // odd groups of [0] <-> even groups of [1]
    auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
    w[0] = t01[0], w[1] = t01[1], w[2] = t23[0], w[3] = t23[1];
}

template <int R, int S, bool PF, int KS, bool WIDE>
__global__ __launch_bounds__(64 * KS * S) void q4_0_matvec_mfma_kernel(MvMfmaDev p) {
    constexpr int kThreads = 64 * KS * S, PD = 16 / KS, kPrefetchCq = PD;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int kc = KS * p.cq * 128;          // features per staged row: cq groups of each wave's share of k
    _Float16 *lds_x = reinterpret_cast<_Float16 *>(lds_raw);                                 // [m][kc], swizzled
    float *red = reinterpret_cast<float *>(lds_raw + (size_t)p.m * kc * sizeof(_Float16));    // [KS S waves][R][4][64]
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = w % KS, st = w / KS;       // this wave's share of the features, its set of rows
    const int b = blockIdx.y, wb = b / p.ratio;
    const int nb = p.k / 32, nit = p.k / 128;
    const int it_lo = q * nit / KS, ni = (q + 1) * nit / KS - it_lo;   // this wave's groups of four blocks
    const _Float16 *act = p.act + (int64_t)b * p.act_stride_b;
    _Float16 *out = p.out + (int64_t)b * p.out_stride_b;
    unsigned char *wave_codes = lds_raw + (size_t)p.m * kc * sizeof(_Float16) + (size_t)KS * S * R * 4 * 64 * sizeof(float) + w * (16 * kCodeRow);   // (WIDE)
    const int arow = min(r16, p.m - 1);      // output rows m..15 of the instruction are never stored: any row serves
    const bool one_chunk = p.nch == 1;

    // Piece v of chunk c: 4 halves of activation row i, quarter qq, group li of the chunk.  A group's 16 vectors of
    // 16 bytes are XOR-swizzled by the row; piece pos of a block goes to vector pos % 4, half pos / 4 of it, so that
    // vector e of a block holds features 4e..4e+3 and 16+4e..16+4e+3.
    auto piece_at = [&](int pc, int li, int qq, int i, int c, const _Float16 *&src, int &dst) -> bool {
        const int lo = qq * nit / KS, have = (qq + 1) * nit / KS - lo, t = c * p.cq + li;
        if (i >= p.m || t >= have) return false;
        src = act + (int64_t)i * p.k + (int64_t)(lo + t) * 128 + pc * 4;
        const int vecg = (pc >> 3) * 4 + (pc & 3), hi = (pc >> 2) & 1;
        dst = i * kc + ((qq * p.cq + li) * 16 + (vecg ^ (i & 15))) * 8 + hi * 4;
        return true;
    };
    // Prefetch mode (PF; cq = kPrefetchCq, at least 512 threads): piece u of a thread is the same 4 halves of row
    // i0 + u * kThreads / 512, so one source pointer and one LDS offset serve all of them.
    const int pf_pc = tid & 31, pf_li = (tid >> 5) & (PD - 1), pf_qq = ((tid >> 5) / PD) & (KS - 1), pf_i0 = tid >> 9;
    const int pf_lo = pf_qq * nit / KS, pf_have = (pf_qq + 1) * nit / KS - pf_lo;
    const _Float16 *pf_src = act + (int64_t)pf_i0 * p.k + (int64_t)(pf_lo + pf_li) * 128 + pf_pc * 4;
    const int pf_vecg = (pf_pc >> 3) * 4 + (pf_pc & 3);
    const int pf_dst = (pf_qq * kPrefetchCq + pf_li) * 128 + ((pf_pc >> 2) & 1) * 4;
    constexpr int kRowStep = kThreads >> 9;

    for (int grp = blockIdx.x; grp < p.groups; grp += gridDim.x) {
        int64_t rows[R];
#pragma unroll
        for (int rr = 0; rr < R; rr++) rows[rr] = (int64_t)wb * p.n + min(((grp * S + st) * R + rr) * 16 + r16, p.n - 1);
        float4_t acc[R];
#pragma unroll
        for (int rr = 0; rr < R; rr++) acc[rr] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

        // PD groups of four blocks per row ahead, across the chunks: the weights do not wait for a chunk's staging.
        u32x4 cn[PD][R];
        // The f16 scales of a round of PD groups come with one load per round: lane group g takes those of group
        // g % PD of the round (8 bytes: four blocks), and ds_bpermute hands them round at use.  (Every load
        // instruction that touches 16 rows costs the compute unit's address path 16 cache lines, whatever it takes
        // from them: without the weights' loads the launch took 61 of 94 us, without the scales' 76.)
        uint64_t sr[R], sr_next[R];
        auto fetch_scales = [&](uint64_t (&dst)[R], int t0) {
            const int t = min(t0 + (g & (PD - 1)), ni - 1);     // (past the end: the last group's again, unused)
#pragma unroll
            for (int rr = 0; rr < R; rr++) dst[rr] = *reinterpret_cast<const uint64_t *>(p.scales + rows[rr] * nb + (it_lo + t) * 4);
        };
        // WIDE: a load instruction takes 128 contiguous bytes (8 blocks: a pair of groups) of 8 rows: lane = (row
        // lane / 8, block lane % 8); slot s of a round holds rows (s & 1) * 8 .. + 7 of pair s / 2.  Half as many cache
        // lines per byte as 64 bytes of 16 rows; the wave passes the pair through its own 16 x 144 bytes of LDS to the
        // lanes that feed the matrix instruction.  Else lane (r, g) loads block g of a group of row r, and the lane
        // groups transpose.
        static_assert(!WIDE || R == 1, "one block of 16 rows per wave");
        const int ra = lane >> 3, b8 = lane & 7;
        int64_t rows_h[2];
#pragma unroll
        for (int h = 0; h < 2; h++) rows_h[h] = (int64_t)wb * p.n + min((grp * S + st) * R * 16 + h * 8 + ra, p.n - 1);
        auto fetch = [&](int slot, int t) {                     // t: the group; WIDE: the pair's first group
            if constexpr (WIDE) {
                const int blk = min((it_lo + t) * 4 + b8, (it_lo + ni) * 4 - 1);   // (an odd share's last pair: the last block again, unused)
                cn[slot][0] = *reinterpret_cast<const u32x4 *>(p.codes + rows_h[slot & 1] * (p.k / 2) + (int64_t)blk * 16);
            } else {
#pragma unroll
                for (int rr = 0; rr < R; rr++)
                    cn[slot][rr] = *reinterpret_cast<const u32x4 *>(p.codes + rows[rr] * (p.k / 2) + (int64_t)((it_lo + t) * 4 + g) * 16);
            }
        };
#pragma unroll
        for (int d = 0; d < PD; d++) {
            const int t = WIDE ? (d & ~1) : d;
            if (t < ni) fetch(d, t);
        }
        if (ni > 0) fetch_scales(sr, 0);
#pragma unroll
        for (int rr = 0; rr < R; rr++) sr_next[rr] = 0;

        const bool stage_here = !one_chunk || grp == (int)blockIdx.x;
        u32x2 held[kStageRegs];
        auto hold = [&](int c) {                                // chunk c's pieces of this thread into registers
            if (c * kPrefetchCq + pf_li < pf_have) {
#pragma unroll
                for (int u = 0; u < kStageRegs; u++)
                    if (pf_i0 + u * kRowStep < p.m)
                        held[u] = *reinterpret_cast<const u32x2 *>(pf_src + (int64_t)u * kRowStep * p.k + c * (kPrefetchCq * 128));
            }
        };
        if constexpr (PF) hold(0);

        for (int c = 0; c < p.nch; c++) {
            if (stage_here) {
                if (c || grp != (int)blockIdx.x) __syncthreads();           // the previous chunk has been read
                if constexpr (PF) {
                    if (c * kPrefetchCq + pf_li < pf_have) {
#pragma unroll
                        for (int u = 0; u < kStageRegs; u++) {
                            const int i = pf_i0 + u * kRowStep;
                            if (i < p.m) *reinterpret_cast<u32x2 *>(lds_x + i * kc + pf_dst + ((pf_vecg ^ (i & 15)) * 8)) = held[u];
                        }
                    }
                } else if (kc == p.k) {
                    // every quarter of k is whole: the one chunk is the rows in their natural order of blocks
                    const int pieces = p.k / 4;
                    for (int v = tid; v < p.m * pieces; v += kThreads) {
                        const int i = v / pieces, cc = v % pieces;
                        const int vec = (cc >> 3) * 4 + (cc & 3), hi = (cc >> 2) & 1;
                        *reinterpret_cast<u32x2 *>(lds_x + i * kc + ((vec ^ (i & 15)) * 8) + hi * 4) =
                            *reinterpret_cast<const u32x2 *>(act + (int64_t)i * p.k + 4 * cc);
                    }
                } else {
                    // piece v = ((i * KS + qq) * cq + li) * 32 + pc for v = tid, tid + kThreads, ...: li and i * KS + qq
                    // are carried along instead of divided out
                    int li = (tid >> 5) % p.cq, iq = (tid >> 5) / p.cq;
                    while (iq < p.m * KS) {
                        const _Float16 *src;
                        int dst;
                        if (piece_at(tid & 31, li, iq % KS, iq / KS, c, src, dst))
                            *reinterpret_cast<u32x2 *>(lds_x + dst) = *reinterpret_cast<const u32x2 *>(src);
                        li += kThreads / 32;
                        while (li >= p.cq) li -= p.cq, iq++;
                    }
                }
                __syncthreads();
                if constexpr (PF)
                    if (c + 1 < p.nch) hold(c + 1);               // in flight during this chunk's arithmetic
            }
            const int cnt = min(max(ni - c * p.cq, 0), p.cq);               // this wave's groups in the chunk
            for (int l0 = 0; l0 < cnt; l0 += PD) {
                if (c * p.cq + l0 + PD < ni) fetch_scales(sr_next, c * p.cq + l0 + PD);
                if constexpr (WIDE) {
#pragma unroll
                for (int pr = 0; pr < PD / 2; pr++) {
                    const int lp = l0 + 2 * pr;
                    if (lp >= cnt) break;
                    const int tp = c * p.cq + lp;                           // even: pairs do not straddle rounds or chunks
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        *reinterpret_cast<u32x4 *>(wave_codes + (h * 8 + ra) * kCodeRow + b8 * 16) = cn[2 * pr + h][0];
                    if (tp + PD < ni) fetch(2 * pr, tp + PD), fetch(2 * pr + 1, tp + PD);
#pragma unroll
                    for (int i2 = 0; i2 < 2; i2++) {
                        const int l = lp + i2;
                        if (l >= cnt) break;
                        const int d = 2 * pr + i2;
                        const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((r16 + 16 * d) * 4, (int)(uint32_t)sr[0]);
                        const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((r16 + 16 * d) * 4, (int)(uint32_t)(sr[0] >> 32));
                        const uint64_t sc = lo | (uint64_t)hi << 32;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int vec = (q * p.cq + l) * 16 + ((j * 4 + g) ^ arow);
                            const half8_t a = *reinterpret_cast<const half8_t *>(lds_x + arow * kc + vec * 8);
                            const uint32_t code = *reinterpret_cast<const uint32_t *>(wave_codes + r16 * kCodeRow + (i2 * 4 + j) * 16 + g * 4);
                            const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, codes_as_halves(code),
                                                                                         float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                            const float dsc = (float)__builtin_bit_cast(_Float16, (uint16_t)(sc >> (16 * j)));
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[0][e] = __builtin_fmaf(dsc, part[e], acc[0][e]);
                        }
                    }
                }
                } else {
#pragma unroll
                for (int d = 0; d < PD; d++) {
                    const int l = l0 + d;
                    if (l >= cnt) break;
                    const int t = c * p.cq + l;                             // t % PD == d: cq is a multiple of PD when nch > 1
                    u32x4 cw[R];
                    uint64_t sc[R];
#pragma unroll
                    for (int rr = 0; rr < R; rr++) {
                        cw[rr] = cn[d][rr];
                        const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((r16 + 16 * d) * 4, (int)(uint32_t)sr[rr]);
                        const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((r16 + 16 * d) * 4, (int)(uint32_t)(sr[rr] >> 32));
                        sc[rr] = lo | (uint64_t)hi << 32;
                    }
                    if (t + PD < ni) fetch(d, t + PD);
#pragma unroll
                    for (int rr = 0; rr < R; rr++) transpose_lane_groups(cw[rr]);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int vec = (q * p.cq + l) * 16 + ((j * 4 + g) ^ arow);
                        const half8_t a = *reinterpret_cast<const half8_t *>(lds_x + arow * kc + vec * 8);
#pragma unroll
                        for (int rr = 0; rr < R; rr++) {
                            const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, codes_as_halves(cw[rr][j]),
                                                                                         float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                            const float dsc = (float)__builtin_bit_cast(_Float16, (uint16_t)(sc[rr] >> (16 * j)));
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[rr][e] = __builtin_fmaf(dsc, part[e], acc[rr][e]);
                        }
                    }
                }
                }
#pragma unroll
                for (int rr = 0; rr < R; rr++) sr[rr] = sr_next[rr];
            }
        }
        // acc[rr][e] = partial out[4 g + e][row rr * 16 + r16] of this wave's set: wave q < 4 of the set adds its KS
        // values of e = q.
        __syncthreads();
#pragma unroll
        for (int rr = 0; rr < R; rr++)
#pragma unroll
            for (int e = 0; e < 4; e++) red[((w * R + rr) * 4 + e) * 64 + lane] = acc[rr][e];
        __syncthreads();
        if (q < 4) {
#pragma unroll
            for (int rr = 0; rr < R; rr++) {
                float sum = 0.0f;
#pragma unroll
                for (int ww = 0; ww < KS; ww++) sum += red[(((st * KS + ww) * R + rr) * 4 + q) * 64 + lane];
                const int i = 4 * g + q, row = ((grp * S + st) * R + rr) * 16 + r16;
                if (i < p.m && row < p.n) out[(int64_t)i * p.n + row] = (_Float16)sum;
            }
        }
    }
}

template <int R, int S, bool PF, int KS, bool WIDE>
int launch_rsp(const MvMfmaDev &p, int64_t act_batch, hipStream_t s) {
    const size_t lds = (size_t)p.m * KS * p.cq * 128 * 2 + (size_t)KS * S * R * 4 * 64 * sizeof(float) + (WIDE ? (size_t)KS * S * 16 * kCodeRow : 0);
    if (lds > 64 * 1024 &&      // beyond the default limit of dynamic LDS: allowed per kernel (and device) on request
        hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_0_matvec_mfma_kernel<R, S, PF, KS, WIDE>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return 2;
    }
    // When the activations fit in LDS a workgroup stages them once and walks several row groups: as many
    // workgroups as are resident at once (by LDS, at most 32 waves per compute unit), each with the same number of groups.
    static const int wg_per_cu = getenv("TROCM_MVM_WG_PER_CU") ? atoi(getenv("TROCM_MVM_WG_PER_CU")) : 0;
    int64_t wgs = p.groups;
    int64_t per_cu = (160 * 1024) / (int64_t)lds;
    if (per_cu > 32 / (KS * S)) per_cu = 32 / (KS * S);
    if (per_cu < 1) per_cu = 1;
    if (wg_per_cu > 0) per_cu = wg_per_cu;
    const int64_t resident = (int64_t)num_compute_units() * per_cu / act_batch;
    if (p.nch == 1 && wgs > resident && resident >= 1) {
        const int64_t turns = (wgs + resident - 1) / resident;
        wgs = (wgs + turns - 1) / turns;
    }
    hipLaunchKernelGGL((q4_0_matvec_mfma_kernel<R, S, PF, KS, WIDE>), dim3((unsigned)wgs, (unsigned)act_batch), dim3(64 * KS * S), lds, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0_matvec (matrix cores) launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <int R, int S, int KS>
int launch_rs(MvMfmaDev p, int64_t act_batch, hipStream_t s) {
    p.groups = (p.n + 16 * R * S - 1) / (16 * R * S);
    constexpr int kThreads = 64 * KS * S;
    if constexpr (kThreads >= 512) {
        static const int allowed = getenv("TROCM_MV_MFMA_PREFETCH") ? atoi(getenv("TROCM_MV_MFMA_PREFETCH")) : 1;
        p.prefetch = allowed && p.nch > 1 && p.cq == 16 / KS && (p.m + (kThreads >> 9) - 1) / (kThreads >> 9) <= kStageRegs;
        if (p.prefetch) return launch_rsp<R, S, true, KS, true>(p, act_batch, s);
    }
    p.prefetch = 0;
    if constexpr (S == 4 && KS == 4)      // (the one shape whose activations may leave no room for the code buffers)
        if (!p.wide) return launch_rsp<R, S, false, KS, false>(p, act_batch, s);
    return launch_rsp<R, S, false, KS, true>(p, act_batch, s);
}

template <int R>
int launch_r(const MvMfmaDev &p, int splits, int sets, int64_t act_batch, hipStream_t s) {
    if (splits == 8) return sets >= 2 ? launch_rs<R, 2, 8>(p, act_batch, s) : launch_rs<R, 1, 8>(p, act_batch, s);
    if (sets == 4) return launch_rs<R, 4, 4>(p, act_batch, s);
    return sets >= 2 ? launch_rs<R, 2, 4>(p, act_batch, s) : launch_rs<R, 1, 4>(p, act_batch, s);
}

}  // namespace

// 2 = not taken (the caller runs the vector-ALU kernel): f32 activations (their products stay in f32 there), k that
// is not a whole number of 128-feature groups, misaligned operands, and the row counts and matrix sizes at which the
// vector-ALU kernel measured faster (up to 3 rows; up to 8 rows against fewer than 2048 weight rows).
int launch_q4_0_matvec_mfma(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                            int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s) {
    static const int enabled = getenv("TROCM_MV_MFMA") ? atoi(getenv("TROCM_MV_MFMA")) : 1;
    static const int forced_min_m = getenv("TROCM_MV_MFMA_MIN_M") ? atoi(getenv("TROCM_MV_MFMA_MIN_M")) : 0;
    static const int forced_lds_kb = getenv("TROCM_MV_MFMA_LDS_KB") ? atoi(getenv("TROCM_MV_MFMA_LDS_KB")) : 0;
    static const int forced_sets = getenv("TROCM_MV_MFMA_SETS") ? atoi(getenv("TROCM_MV_MFMA_SETS")) : 0;
    if (!enabled || act_dtype != TROCM_F16 || m < 2 || m > 16 || k % 128 != 0 || k < 128) return 2;
    if ((uintptr_t)codes % 16 || (uintptr_t)scales % 8 || (uintptr_t)act % 8 || (uintptr_t)out % 2) return 2;
    if (n < 1 || n >= (1ll << 30) || k >= (1ll << 30) || act_batch < 1 || act_batch > 65535) return 2;
    const int64_t cus = num_compute_units();
    const int64_t blocks16 = (n + 15) / 16 * act_batch;          // blocks of 16 weight rows in the launch
    // Measured against the vector-ALU kernel (us; 14336 x 4096: 3 rows 12.1 vs 13.2, 4 rows 12.5 vs 16.7, 8 rows 13.6 vs
    // 38.8; 4096 x 4096: 3 rows 6.4 vs 6.0, 4 rows 6.8 vs 6.9, 8 rows 8.3 vs 14.2; 128256 x 4096: 3 rows 80.5 vs 78.2,
    // 4 rows 78 vs 98; 1024 x 4096, 8 rows: 10.1 vs 7.4).
    const int64_t min_m = forced_min_m > 0 ? forced_min_m : 4;
    if (m < min_m || (m <= 8 && forced_min_m == 0 && blocks16 * 2 < cus)) return 2;
    MvMfmaDev p;
    memset(&p, 0, sizeof(p));
    p.codes = (const uint8_t *)codes, p.scales = (const uint16_t *)scales;
    p.act = (const _Float16 *)act, p.out = (_Float16 *)out;
    p.act_stride_b = m * k, p.out_stride_b = m * n;
    p.n = (int)n, p.k = (int)k, p.m = (int)m, p.ratio = (int)(act_batch / w_batch);
    // Every wave walks one share of k: a quarter, or an eighth when the matrix has too few rows to give every SIMD a
    // wave otherwise.
    static const int forced_cq = getenv("TROCM_MV_MFMA_CQ") ? atoi(getenv("TROCM_MV_MFMA_CQ")) : 0;
    static const int forced_splits = getenv("TROCM_MV_MFMA_SPLITS") ? atoi(getenv("TROCM_MV_MFMA_SPLITS")) : 0;
    int splits = blocks16 < 2 * cus && k >= 2048 ? 8 : 4;
    if (forced_splits == 4 || forced_splits == 8) splits = forced_splits;
    const int64_t per_split = (k / 128 + splits - 1) / splits;
    // One block of 16 rows per wave (R = 1; two, sharing each read of the activations, measured slower: 105 vs 91 us
    // for 128256 x 4096 and 8 rows, and are not instantiated).  Sets of waves behind one staged chunk: one of 8 waves
    // for matrices of few rows; of 4 waves, four when that still leaves about a workgroup per compute unit (14336
    // rows, 8 activation rows: 15.2 us; two sets 16.6 us; one 21.8 us), else two.
    int sets = splits == 8 ? 1 : blocks16 >= 3 * cus ? 4 : 2;
    if (forced_sets == 1 || forced_sets == 2 || forced_sets == 4) sets = forced_sets;
    // If the whole of the activations fits the LDS budget they are staged once per workgroup; else in chunks of 2048
    // features (512 or 256 of every share, a multiple of the weights' prefetch depth), the next chunk waiting in
    // registers.  Budget: what leaves room for two workgroups of 8 waves or one of 16 on a compute unit beside the
    // partial sums and the waves' code buffers; all of the LDS when every workgroup walks many row groups behind one
    // staging (128256 x 4096 with 16 rows: 95 us, in chunks 125 us; 14336 x 4096: 20.0 us, in chunks 16.5 us), with
    // without the code buffers if that is what makes it fit.
    const int64_t x_bytes = m * splits * per_split * 128 * 2;
    auto beside = [&](int st, bool wide = true) { return (int64_t)splits * st * (4 * 64 * 4 + (wide ? 16 * kCodeRow : 0)); };
    const int64_t lds_all = 160 * 1024;
    const bool walks_many = blocks16 / 4 >= 4 * cus;
    // (16 activation rows of 4096 features leave the 16 waves no room for code buffers: the 64-byte loads then)
    p.wide = !(walks_many && splits * sets == 16 && x_bytes + beside(sets) > lds_all && x_bytes + beside(sets, false) <= lds_all);
    const int64_t budget = forced_lds_kb > 0 ? (int64_t)forced_lds_kb * 1024
                         : walks_many        ? lds_all - beside(sets, p.wide)
                         : splits * sets >= 16 ? 64 * 1024 : lds_all / 2 - beside(sets);
    if (x_bytes <= budget) {
        p.cq = (int)per_split, p.nch = 1;
    } else {
        const int pd = 16 / splits;
        p.cq = forced_cq > 0 && forced_cq % pd == 0 ? forced_cq : pd;
        p.nch = (int)((per_split + p.cq - 1) / p.cq);
    }
    if (p.nch > 1 && m > 8 && forced_sets == 0) sets = splits == 8 ? 2 : 4;    // 1024 threads hold a chunk of 16 rows in their registers
    return launch_r<1>(p, splits, sets, act_batch, s);
}

}  // namespace trocm
