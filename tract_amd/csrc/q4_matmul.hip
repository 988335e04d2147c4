// Q4_0 weights x many activation rows on the matrix cores (the prefill-time projection): gfx950.
//
//   out[b, i, j] = sum_k act[b, i, k] * dequant(W[b / ratio, j, k]),   i < m,  m > 8,  f16 activations
//
// the matrix-matrix arm of GgmlGemm (cuda/src/kernels/matmul/mod.rs:605-610: m > 8 goes to
// dispatch_ggml_matmul_q40, whose kernel quantises the activations to Q8_1 and takes integer dot products).  This
// kernel computes what the operator's own test compares against (mod.rs:864-890): the product with the weights
// dequantised to f16 -- (code - 8) * d rounded once to f16, the value dequant_block_f16 stores (q4_0.rs:82-95) --
// accumulated in f32.
//
// C^T[n, m] = W[n, k] . act^T[k, m] with v_mfma_f32_32x32x16_f16: both operands are rows of k, so every fragment
// is one 128-bit LDS read.  A workgroup of 4 waves owns a 128 x 128 tile of C^T (each wave 64 x 64: four
// accumulators; 128 x 64 with two accumulators per wave when the larger tiles would be fewer than the compute units), walks k in chunks of 64 (two quantisation blocks), and keeps the next chunk in registers while
// it multiplies the current one: a thread fetches the 16 code bytes and the scale of one weight block and four
// 16-byte pieces of the activations, dequantises its block on the way into LDS (one v_perm per two codes puts the
// nibble under the exponent byte 0x64: 1024 + u; minus 1032 is exact; times d rounds once).
//
// Roofline: MFMA-bound for the m of a prefill chunk (2 m n k flops over n k / 2 + 2 m k + 2 m n bytes).
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kMmThreads = 256;
constexpr int BN = 128, BK = 64;   // (the tile's m extent BM is 128, or 64 when 128 would leave compute units without a tile)
constexpr int ROW = BK + 8;   // halves per tile row in LDS: the 16 rows of a 128-bit read pass fall into 16 distinct bank groups

struct MatMulDev {
    const uint8_t *codes;     // [w_batch, n, k/2]; TILED: [w_batch, n / 16, k / 128] records of 1152 bytes (q4_tiled.hip)
    const uint16_t *scales;   // [w_batch, n, k/32]; TILED: unused (the scales are in the records)
    const _Float16 *act;      // [act_batch, m, k]
    _Float16 *out;            // [act_batch, m, n]
    int n, k, m, ratio;       // ratio = act_batch / w_batch
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// four code nibbles (one per byte of w) -> their dequantised f16 values, two words
__device__ __forceinline__ void dequant4(uint32_t w, half2_t d2, uint32_t &lo, uint32_t &hi) {
    const half2_t zero = {(_Float16)1032.0f, (_Float16)1032.0f};   // 1024 + 8
    lo = __builtin_bit_cast(uint32_t, (as_half2(perm(0x64646464u, w, 0x04010400u)) - zero) * d2);
    hi = __builtin_bit_cast(uint32_t, (as_half2(perm(0x64646464u, w, 0x04030402u)) - zero) * d2);
}

template <int BM, bool TILED>
__global__ __launch_bounds__(kMmThreads, 2) void q4_0_matmul_kernel(MatMulDev p) {
    constexpr int MJ = BM / 64;        // 32-row halves of m per wave: the wave's corner is 64 (n) x 32 MJ (m)
    constexpr int AP = BM * 8 / kMmThreads;   // 16-byte activation pieces per thread and chunk
    __shared__ __attribute__((aligned(16))) _Float16 lds_w[2][BN * ROW];
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][BM * ROW];

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hb = lane >> 5, l32 = lane & 31;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM, b = blockIdx.z, wb = b / p.ratio;
    const int wn = 64 * (w & 1), wm = 32 * MJ * (w >> 1);   // this wave's corner of the tile
    const int nb = p.k / 32;

    // staging roles: weight block (row tid / 2, block tid % 2 of the chunk); activation pieces j * 256 + tid
    const int w_row = tid >> 1, w_blk = tid & 1;
    const int64_t w_grow = (int64_t)wb * p.n + min(n0 + w_row, p.n - 1);   // rows past the end repeat the last one
    const uint8_t *w_codes = p.codes + w_grow * (p.k / 2) + w_blk * 16;
    const uint16_t *w_scales = p.scales + w_grow * nb + w_blk;
    const _Float16 *a_base = p.act + (int64_t)b * p.m * p.k;
    int a_row[AP], a_col[AP];
#pragma unroll
    for (int j = 0; j < AP; j++) {
        const int c = j * kMmThreads + tid;
        a_row[j] = c >> 3, a_col[j] = (c & 7) * 8;
    }

    // TILED: a chunk is one half (blocks 2 hh, 2 hh + 1) of a tile of each of the 8 row groups of the workgroup's 128
    // rows; this thread stages slot `lane` (row lane % 16, bytes 4 g .. 4 g + 3 of each block, g = lane / 16) of row
    // groups w and w + 4: 8 bytes of codes and two scales each.
    const int t_r = lane & 15, t_g = lane >> 4;
    const uint8_t *t_rec[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int64_t grp = (int64_t)wb * (p.n / 16) + min(n0 / 16 + w + 4 * h, p.n / 16 - 1);   // groups past the end repeat the last one
        t_rec[h] = p.codes + grp * (p.k / 128) * 1152;
    }
    u32x2 tpre[2];
    uint32_t tspre[2];

    u32x4 cpre, apre[AP];
    uint16_t spre;
    auto prefetch = [&](int k0) {
        if constexpr (TILED) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint8_t *rec = t_rec[h] + (int64_t)(k0 / 128) * 1152;
                tpre[h] = *reinterpret_cast<const u32x2 *>(rec + 16 * lane + 8 * ((k0 / 64) & 1));
                tspre[h] = *reinterpret_cast<const uint32_t *>(rec + 1024 + 8 * t_r + 4 * ((k0 / 64) & 1));
            }
        } else {
            cpre = *reinterpret_cast<const u32x4 *>(w_codes + (k0 / 32) * 16);
            spre = w_scales[k0 / 32];
        }
#pragma unroll
        for (int j = 0; j < AP; j++)
            apre[j] = *reinterpret_cast<const u32x4 *>(a_base + (int64_t)min(m0 + a_row[j], p.m - 1) * p.k + k0 + a_col[j]);
    };
    auto stage = [&](int buf) {
        if constexpr (TILED) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int jj = 0; jj < 2; jj++) {
                    const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t)(tspre[h] >> (16 * jj)));
                    const half2_t d2 = {d, d};
                    const uint32_t word = tpre[h][jj];
                    uint32_t lo0, lo1, hi0, hi1;   // elements 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3 of block jj of the chunk
                    dequant4(word & 0x0F0F0F0Fu, d2, lo0, lo1);
                    dequant4((word >> 4) & 0x0F0F0F0Fu, d2, hi0, hi1);
                    _Float16 *dst = &lds_w[buf][((w + 4 * h) * 16 + t_r) * ROW + jj * 32 + 4 * t_g];
                    *reinterpret_cast<u32x2 *>(dst) = u32x2{lo0, lo1};
                    *reinterpret_cast<u32x2 *>(dst + 16) = u32x2{hi0, hi1};
                }
        } else {
        const _Float16 d = __builtin_bit_cast(_Float16, spre);
        const half2_t d2 = {d, d};
        const uint32_t cw[4] = {cpre.x, cpre.y, cpre.z, cpre.w};
        uint32_t lo[8], hi[8];   // elements 0..15 (low nibbles) and 16..31 (high nibbles) of the block, two per word
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dequant4(cw[i] & 0x0F0F0F0Fu, d2, lo[2 * i], lo[2 * i + 1]);
            dequant4((cw[i] >> 4) & 0x0F0F0F0Fu, d2, hi[2 * i], hi[2 * i + 1]);
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(&lds_w[buf][w_row * ROW + w_blk * 32]);
        dst[0] = u32x4{lo[0], lo[1], lo[2], lo[3]};
        dst[1] = u32x4{lo[4], lo[5], lo[6], lo[7]};
        dst[2] = u32x4{hi[0], hi[1], hi[2], hi[3]};
        dst[3] = u32x4{hi[4], hi[5], hi[6], hi[7]};
        }
#pragma unroll
        for (int j = 0; j < AP; j++) *reinterpret_cast<u32x4 *>(&lds_a[buf][a_row[j] * ROW + a_col[j]]) = apre[j];
    };

    float16_t acc[2][MJ];   // [n half][m half] of the wave's corner
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < MJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int n_chunks = p.k / BK;
    prefetch(0);
    stage(0);
    if (n_chunks > 1) prefetch(BK);
    for (int it = 0; it < n_chunks; it++) {
        __syncthreads();   // chunk `it` is in LDS; every wave is done with the buffer about to be overwritten
        const int cur = it & 1;
        if (it + 1 < n_chunks) {
            stage(cur ^ 1);
            if (it + 2 < n_chunks) prefetch((it + 2) * BK);
        }
        const _Float16 *wt = &lds_w[cur][(wn + l32) * ROW + 8 * hb];
        const _Float16 *at = &lds_a[cur][(wm + l32) * ROW + 8 * hb];
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8_t wf[2], af[MJ];
#pragma unroll
            for (int i = 0; i < 2; i++) wf[i] = *reinterpret_cast<const half8_t *>(wt + (32 * i) * ROW + 16 * ks);
#pragma unroll
            for (int j = 0; j < MJ; j++) af[j] = *reinterpret_cast<const half8_t *>(at + (32 * j) * ROW + 16 * ks);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < MJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[i], af[j], acc[i][j], 0, 0, 0);
        }
    }

    // C^T[n, m]: register r of a lane is n = 8 (r / 4) + 4 hb + r % 4 of the 32 x 32 tile, m = lane % 32
    _Float16 *out = p.out + (int64_t)b * p.m * p.n;
    const bool vec = (p.n % 4) == 0;
#pragma unroll
    for (int j = 0; j < MJ; j++) {
        const int mi = m0 + wm + 32 * j + l32;
        if (mi >= p.m) continue;
        _Float16 *orow = out + (int64_t)mi * p.n;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                const int ni = n0 + wn + 32 * i + 8 * rq + 4 * hb;
                half4_t h4;
#pragma unroll
                for (int e = 0; e < 4; e++) h4[e] = (_Float16)acc[i][j][4 * rq + e];
                if (vec && ni + 3 < p.n) {
                    *reinterpret_cast<half4_t *>(orow + ni) = h4;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (ni + e < p.n) orow[ni + e] = h4[e];
                }
            }
    }
}

}  // namespace

// 2 = not taken (the caller runs the rows in groups of 8 on the vector-ALU kernel): f32 activations (their products
// stay in f32 there), k that is not a whole number of 64-element chunks, misaligned operands.
int launch_q4_0_matmul(const void *codes, const void *scales, int64_t w_batch, int64_t n, int64_t k, const void *act,
                       int act_dtype, int64_t act_batch, int64_t m, void *out, hipStream_t s, int tiled) {
    static const int enabled = getenv("TROCM_Q4_MATMUL") ? atoi(getenv("TROCM_Q4_MATMUL")) : 1;
    if (!enabled || act_dtype != TROCM_F16 || m <= 8 || k % BK != 0) return 2;
    if ((uintptr_t)codes % 16 || (uintptr_t)act % 16 || (uintptr_t)out % 8) return 2;
    if (n >= (1ll << 30) || m >= (1ll << 30) || k >= (1ll << 30) || act_batch > 65535) return 2;
    MatMulDev p;
    memset(&p, 0, sizeof(p));
    p.codes = (const uint8_t *)codes, p.scales = (const uint16_t *)scales;
    p.act = (const _Float16 *)act, p.out = (_Float16 *)out;
    p.n = (int)n, p.k = (int)k, p.m = (int)m, p.ratio = (int)(act_batch / w_batch);
    // 128 x 128 tiles unless they are fewer than the compute units: then 128 (n) x 64 (m), twice as many workgroups
    const int64_t gx = (n + BN - 1) / BN;
    const bool half_m = gx * ((m + 127) / 128) * act_batch < num_compute_units() && m > 64;
    const int64_t gy = half_m ? (m + 63) / 64 : (m + 127) / 128;
    if (gy > 65535) return 2;
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)act_batch);
    if (tiled && half_m)
        hipLaunchKernelGGL((q4_0_matmul_kernel<64, true>), grid, dim3(kMmThreads), 0, s, p);
    else if (tiled)
        hipLaunchKernelGGL((q4_0_matmul_kernel<128, true>), grid, dim3(kMmThreads), 0, s, p);
    else if (half_m)
        hipLaunchKernelGGL((q4_0_matmul_kernel<64, false>), grid, dim3(kMmThreads), 0, s, p);
    else
        hipLaunchKernelGGL((q4_0_matmul_kernel<128, false>), grid, dim3(kMmThreads), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0_matmul launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace trocm
