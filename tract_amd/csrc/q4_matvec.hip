// Q4_0 weights x activations, few activation rows (the decode-time projection): gfx950.
//
//   out[b, i, j] = sum_k act[b, i, k] * dequant(W[b / ratio, j, k]),   i < m <= 8
//
// the matrix-vector arm of GgmlGemm (cuda/src/kernels/matmul/mod.rs:575-627, m <= 8 at :605-606,
// launch geometry :481-529).  The reference kernel quantises the activations to Q8_1 and takes
// integer dot products; its own test holds it, loosely, to the CPU result of the dequantised
// weights (mod.rs:864-890).  This kernel computes that definition directly: the weights'
// codes become exact small integers in f16 (or f32), the products accumulate in f32, and each
// block's sum is scaled by its f16 scale once.
//
// Layout: the canonical 18-byte blocks are split at load time into a code plane [rows, k/2] (a
// block's 16 bytes stay together: low nibbles are elements 0..15, high nibbles 16..31) and a
// scale plane [rows, k/32] of f16 -- the planes of a Q4_0 KV cache -- so that a wave reads a row
// with coalesced 128-bit loads (consecutive lanes, consecutive blocks).
//
// Work: one workgroup of 4 waves, each wave R output rows at a time; lane l takes blocks l, l+64, ...
// of the current k chunk, whose activations sit in LDS (read once per lane and block, used for R
// rows).  Accumulators are reduced across the wave at the end.
//
// Roofline: HBM-bound on the weights: 18 bytes per 32 weights, read once.  (From about 4 f16 rows on the arithmetic
// of this kernel, which repeats per row, takes longer than the weights: those calls go to q4_matvec_mfma.hip.)
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMvWaves = 4, kMvThreads = 64 * kMvWaves;
constexpr int kLdsBytes = 32 * 1024;   // activation chunk in LDS

struct MatVecDev {
    const uint8_t *codes;     // [w_batch, n, k/2]
    const uint16_t *scales;   // [w_batch, n, k/32]
    const void *act;          // [act_batch, m, k]
    void *out;                // [act_batch, m, n]
    int64_t act_stride_b, out_stride_b;   // elements between consecutive batches of act and out
    int n, k, ratio;          // ratio = act_batch / w_batch
    int kc;                   // activations staged per chunk (elements of k), a multiple of 32
    int groups;               // row groups of kMvWaves * R rows
};

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
// bytes (b0, b1) / (b2, b3) of a word of 4-bit codes as the halves (1024 + b): 0x6400 | b
__device__ __forceinline__ half2_t magic_lo(uint32_t c4) { return as_half2(perm(0x64646464u, c4, 0x04010400u)); }
__device__ __forceinline__ half2_t magic_hi(uint32_t c4) { return as_half2(perm(0x64646464u, c4, 0x04030402u)); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float readlane_f(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_f<0x128>(x);   // row_ror:8, 4, 2, 1 within rows of 16 lanes
    x += dpp_f<0x124>(x);
    x += dpp_f<0x122>(x);
    x += dpp_f<0x121>(x);
    return (readlane_f(x, 0) + readlane_f(x, 16)) + (readlane_f(x, 32) + readlane_f(x, 48));
}

template <typename T>
__device__ __forceinline__ T out_cast(float x);
template <>
__device__ __forceinline__ __half out_cast<__half>(float x) { return __float2half_rn(x); }
template <>
__device__ __forceinline__ float out_cast<float>(float x) { return x; }

// sum over one block of (code - 8) * x for M activation rows, f16 activations in LDS
template <int M>
__device__ __forceinline__ void block_dot(const u32x4 c, const half2_t (&x2)[M][16], float (&acc)[M]) {
    const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
    const half2_t eight = {(_Float16)1032.0f, (_Float16)1032.0f};
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t lo = cw[w] & 0x0F0F0F0Fu, hi = (cw[w] >> 4) & 0x0F0F0F0Fu;
        // elements 4w, 4w+1 | 4w+2, 4w+3 | 16+4w, 16+4w+1 | 16+4w+2, 16+4w+3 as exact integers code - 8
        const half2_t e0 = magic_lo(lo) - eight, e1 = magic_hi(lo) - eight, e2 = magic_lo(hi) - eight, e3 = magic_hi(hi) - eight;
#pragma unroll
        for (int i = 0; i < M; i++) {
            acc[i] = __builtin_amdgcn_fdot2(e0, x2[i][2 * w], acc[i], false);
            acc[i] = __builtin_amdgcn_fdot2(e1, x2[i][2 * w + 1], acc[i], false);
            acc[i] = __builtin_amdgcn_fdot2(e2, x2[i][8 + 2 * w], acc[i], false);
            acc[i] = __builtin_amdgcn_fdot2(e3, x2[i][8 + 2 * w + 1], acc[i], false);
        }
    }
}

// the same for f32 activations: codes to f32 one byte at a time, fma in f32
template <int M>
__device__ __forceinline__ void block_dot(const u32x4 c, const float (&x)[M][32], float (&acc)[M]) {
    const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t lo = cw[w] & 0x0F0F0F0Fu, hi = (cw[w] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float fl = (float)((lo >> (8 * j)) & 0xffu) - 8.0f, fh = (float)((hi >> (8 * j)) & 0xffu) - 8.0f;
#pragma unroll
            for (int i = 0; i < M; i++) {
                acc[i] = __builtin_fmaf(fl, x[i][4 * w + j], acc[i]);
                acc[i] = __builtin_fmaf(fh, x[i][16 + 4 * w + j], acc[i]);
            }
        }
    }
}

template <typename T, int M, int R>
__global__ __launch_bounds__(kMvThreads) void q4_0_matvec_kernel(MatVecDev p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    T *lds_x = reinterpret_cast<T *>(lds_raw);          // [M][kc]
    constexpr bool F16 = sizeof(T) == 2;
    constexpr int EPV = 16 / sizeof(T), VPB = 32 / EPV; // elements per 16-byte vector, vectors per block
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = blockIdx.y, wb = b / p.ratio;
    const int nb = p.k / 32;                            // blocks per weight row
    const T *act = reinterpret_cast<const T *>(p.act) + (int64_t)b * p.act_stride_b;
    T *out = reinterpret_cast<T *>(p.out) + (int64_t)b * p.out_stride_b;
    const bool one_chunk = p.kc >= p.k;                 // the activations fit in LDS: staged once per workgroup

    // A workgroup takes row groups g, g + gridDim.x, ... (kMvWaves * R rows each).
    for (int g = blockIdx.x; g < p.groups; g += gridDim.x) {
        const int row0 = (g * kMvWaves + w) * R;        // first output column of this wave
        // Row indices only (pointers are formed at each fetch): 2R pointers held across the loop cost
        // more scalar registers than the kernel has.
        int rows[R];
#pragma unroll
        for (int r = 0; r < R; r++) rows[r] = wb * p.n + min(row0 + r, p.n - 1);   // rows past the end repeat the last one
        float acc[R][M];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int i = 0; i < M; i++) acc[r][i] = 0.0f;

        for (int k0 = 0; k0 < p.k; k0 += p.kc) {
            const int kn = min(p.kc, p.k - k0);         // a multiple of 32
            const int cb = kn / 32, b0 = k0 / 32;       // blocks in this chunk, first block
            u32x4 cn[R];
            uint16_t scn[R];
            auto fetch = [&](int blk) {                 // this lane's block of each of the R rows
#pragma unroll
                for (int r = 0; r < R; r++) {
                    cn[r] = *reinterpret_cast<const u32x4 *>(p.codes + (int64_t)rows[r] * (p.k / 2) + (int64_t)(b0 + blk) * 16);
                    scn[r] = p.scales[(int64_t)rows[r] * nb + b0 + blk];
                }
            };
            if (lane < cb) fetch(lane);                 // in flight while the activations are staged
            if (!one_chunk || g == (int)blockIdx.x) {
                if (k0) __syncthreads();
                // stage act[:, k0 .. k0+kn) -> lds_x[i][0 .. kn).  The 16-byte vectors of a block are rotated
                // by block * VPB / 16, so that the 16 lanes of a 128-bit LDS read pass (16 consecutive
                // blocks) fall into 16 different bank groups.
                const int vec_per_row = kn / EPV;
                for (int v = tid; v < M * vec_per_row; v += kMvThreads) {
                    const int i = v / vec_per_row, c = v % vec_per_row;
                    const int blk = c / VPB, ch = c % VPB;
                    *reinterpret_cast<u32x4 *>(lds_x + (int64_t)i * p.kc + (blk * VPB + ((ch + blk * VPB / 16) & (VPB - 1))) * EPV) =
                        *reinterpret_cast<const u32x4 *>(act + (int64_t)i * p.k + k0 + c * EPV);
                }
                __syncthreads();
            }
            for (int blk = lane; blk < cb; blk += 64) {
                u32x4 c[R];
                uint16_t sc[R];
#pragma unroll
                for (int r = 0; r < R; r++) c[r] = cn[r], sc[r] = scn[r];
                if (blk + 64 < cb) fetch(blk + 64);     // the next block's weights are in flight during this one's arithmetic
                if constexpr (F16) {
                    half2_t x2[M][16];
#pragma unroll
                    for (int i = 0; i < M; i++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const u32x4 xv = *reinterpret_cast<const u32x4 *>(lds_x + (int64_t)i * p.kc + blk * 32 + ((v + blk / 4) & 3) * 8);
                            x2[i][4 * v] = as_half2(xv.x), x2[i][4 * v + 1] = as_half2(xv.y);
                            x2[i][4 * v + 2] = as_half2(xv.z), x2[i][4 * v + 3] = as_half2(xv.w);
                        }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        float part[M];
#pragma unroll
                        for (int i = 0; i < M; i++) part[i] = 0.0f;
                        block_dot<M>(c[r], x2, part);
                        const float d = __half2float(__ushort_as_half(sc[r]));
#pragma unroll
                        for (int i = 0; i < M; i++) acc[r][i] = __builtin_fmaf(d, part[i], acc[r][i]);
                    }
                } else {
                    float x[M][32];
#pragma unroll
                    for (int i = 0; i < M; i++)
#pragma unroll
                        for (int v = 0; v < 8; v++) {
                            const float4_t xv = *reinterpret_cast<const float4_t *>(lds_x + (int64_t)i * p.kc + blk * 32 + ((v + blk / 2) & 7) * 4);
                            x[i][4 * v] = xv[0], x[i][4 * v + 1] = xv[1], x[i][4 * v + 2] = xv[2], x[i][4 * v + 3] = xv[3];
                        }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        float part[M];
#pragma unroll
                        for (int i = 0; i < M; i++) part[i] = 0.0f;
                        block_dot<M>(c[r], x, part);
                        const float d = __half2float(__ushort_as_half(sc[r]));
#pragma unroll
                        for (int i = 0; i < M; i++) acc[r][i] = __builtin_fmaf(d, part[i], acc[r][i]);
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int i = 0; i < M; i++) {
                const float sum = wave_sum(acc[r][i]);
                if (lane == 0 && row0 + r < p.n) out[(int64_t)i * p.n + row0 + r] = out_cast<T>(sum);
            }
    }
}

template <typename T, int M, int R>
int launch_mr(const MatVecDev &p, int64_t act_batch, hipStream_t s) {
    const int rows_per_wg = kMvWaves * R;
    MatVecDev q = p;
    q.groups = (p.n + rows_per_wg - 1) / rows_per_wg;
    // When the activations fit in LDS a workgroup stages them once and walks several row groups:
    // about 8 workgroups per compute unit are resident, more would only repeat the staging.
    static const int wg_per_cu = getenv("TROCM_MV_WG_PER_CU") ? atoi(getenv("TROCM_MV_WG_PER_CU")) : 8;
    int64_t wgs = q.groups;
    const int64_t resident = (int64_t)num_compute_units() * wg_per_cu / act_batch;
    if (q.kc >= q.k && wgs > resident && resident >= 1) wgs = resident;
    dim3 grid((unsigned)wgs, (unsigned)act_batch);
    const size_t lds = (size_t)M * q.kc * sizeof(T);
    hipLaunchKernelGGL((q4_0_matvec_kernel<T, M, R>), grid, dim3(kMvThreads), lds, s, q);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0_matvec launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_m(const MatVecDev &p, int m, int64_t act_batch, hipStream_t s) {
    // Rows per wave: four share each activation read; fewer when that would leave compute units idle.
    static const int forced_rows = getenv("TROCM_MV_ROWS") ? atoi(getenv("TROCM_MV_ROWS")) : 0;
    const int64_t wgs4 = (p.n + 4 * kMvWaves - 1) / (4 * kMvWaves) * act_batch;
    int rows = wgs4 >= 4 * (int64_t)num_compute_units() ? 4 : wgs4 >= 2 * (int64_t)num_compute_units() ? 2 : 1;
    if (forced_rows == 1 || forced_rows == 2 || forced_rows == 4) rows = forced_rows;
    if (m == 1) return rows == 4 ? launch_mr<T, 1, 4>(p, act_batch, s) : rows == 2 ? launch_mr<T, 1, 2>(p, act_batch, s) : launch_mr<T, 1, 1>(p, act_batch, s);
    if (m == 2) return rows == 4 ? launch_mr<T, 2, 4>(p, act_batch, s) : rows == 2 ? launch_mr<T, 2, 2>(p, act_batch, s) : launch_mr<T, 2, 1>(p, act_batch, s);
    switch (m) {
        case 3: return launch_mr<T, 3, 2>(p, act_batch, s);
        case 4: return launch_mr<T, 4, 2>(p, act_batch, s);
        case 5: return launch_mr<T, 5, 1>(p, act_batch, s);
        case 6: return launch_mr<T, 6, 1>(p, act_batch, s);
        case 7: return launch_mr<T, 7, 1>(p, act_batch, s);
        case 8: return launch_mr<T, 8, 1>(p, act_batch, s);
    }
    return fail("q4_0_matvec: m = %d activation rows (1..8 are handled here)", m);
}

}  // namespace

int launch_q4_0_matvec(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                       int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s) {
    const int64_t es = (int64_t)elem_bytes(act_dtype);
    if (m >= 2 && m <= 16) {   // a few f16 rows: 16 weight rows x 16 activation rows per matrix instruction (q4_matvec_mfma.hip)
        const int rc = launch_q4_0_matvec_mfma(codes, scales, w_batch, n, k, act, act_dtype, act_batch, m, out, s);
        if (rc != 2) return rc;
    }
    if (m > 8) {   // the matrix-matrix arm (q4_matmul.hip) for f16 activations
        const int rc = launch_q4_0_matmul(codes, scales, w_batch, n, k, act, act_dtype, act_batch, m, out, s);
        if (rc != 2) return rc;
    }
    // What it does not take runs as groups of 8 rows (each group streams the weights once): correct
    // for any m, efficient only for the few rows of a decode step.
    for (int64_t i0 = 0; i0 < m; i0 += 8) {
        const int64_t mg = m - i0 < 8 ? m - i0 : 8;
        MatVecDev p;
        memset(&p, 0, sizeof(p));
        p.codes = (const uint8_t *)codes, p.scales = (const uint16_t *)scales;
        p.act = (const char *)act + i0 * k * es, p.out = (char *)out + i0 * n * es;
        p.act_stride_b = m * k, p.out_stride_b = m * n;
        p.n = (int)n, p.k = (int)k, p.ratio = (int)(act_batch / w_batch);
        int64_t kc = kLdsBytes / (mg * es) / 32 * 32;   // what fits, in whole blocks
        if (kc > k) kc = k;
        p.kc = (int)kc;
        const int rc = act_dtype == TROCM_F16 ? launch_m<__half>(p, (int)mg, act_batch, s) : launch_m<float>(p, (int)mg, act_batch, s);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace trocm
