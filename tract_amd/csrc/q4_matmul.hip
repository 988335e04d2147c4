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
// C^T[n, m] = W[n, k] . act^T[k, m] with v_mfma_f32_32x32x16_f16, two kernels:
// * weights held as planes of codes and scales (q4_0_matmul_kernel): both operands are rows of k in LDS, every fragment
//   one 128-bit LDS read.  A workgroup of 4 waves owns a 128 x 128 tile of C^T (each wave 64 x 64: four accumulators;
//   128 x 64 with two accumulators per wave when the larger tiles would be fewer than the compute units), walks k in
//   chunks of 64 (two quantisation blocks), and keeps the next chunk in registers while it multiplies the current one: a
//   thread fetches the 16 code bytes and the scale of one weight block and four 16-byte pieces of the activations,
//   dequantises its block on the way into LDS (one v_perm per two codes puts the nibble under the exponent byte 0x64:
//   1024 + u; minus 1032 is exact; times d rounds once).
// * weights held as tiles (q4_0_tiled_matmul_kernel, further down): the weight fragments come straight from the records
//   into registers; only the activations pass through LDS.
//
// Roofline: MFMA-bound for the m of a prefill chunk (2 m n k flops over n k / 2 + 2 m k + 2 m n bytes).
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include <type_traits>
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
    const uint8_t *codes;     // [w_batch, n, k/2]; tiled weights: [w_batch, n / 16, k / 128] records of 1152 bytes (q4_tiled.hip)
    const uint16_t *scales;   // [w_batch, n, k/32]; tiled weights: unused (the scales are in the records)
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

template <int BM>
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

    u32x4 cpre, apre[AP];
    uint16_t spre;
    auto prefetch = [&](int k0) {
        cpre = *reinterpret_cast<const u32x4 *>(w_codes + (k0 / 32) * 16);
        spre = w_scales[k0 / 32];
#pragma unroll
        for (int j = 0; j < AP; j++)
            apre[j] = *reinterpret_cast<const u32x4 *>(a_base + (int64_t)min(m0 + a_row[j], p.m - 1) * p.k + k0 + a_col[j]);
    };
    auto stage = [&](int buf) {
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

// ---- tiled weights, fragments straight from the records -----------------------------------------------------------------
// The weights never pass through LDS: slot (r, g) of a record holds, for each of the tile's 4 blocks, the 8 codes of row r
// that one lane contributes to a contraction of 16 (elements 4g..4g+3 and 16+4g..16+4g+3 of the block), so lane
// (row = lane % 32, half = lane / 32) of v_mfma_f32_32x32x16_f16 takes slots g = half and g = 2 + half of its row's
// record -- two 128-bit loads per tile and 32 rows -- and dequantises them in registers ((1024 + code) - 1032, times d,
// rounded once: the value dequant_block_f16 stores).  The order of the features inside a contraction does not matter
// as long as both operands agree: the activations are staged with vector v = 4 block + g of a row holding the same
// eight features.  A workgroup of 4 waves owns 128 NI (n) x BM (m) of C^T, each wave 32 NI x BM: with NI = 2 an
// activation fragment read from LDS feeds two matrix instructions and a dequantised weight fragment BM / 32, so LDS
// moves half a fragment per instruction (the kernel above: one, which is all LDS can deliver).  BM = 64 and then NI = 1 are
// for launches that would otherwise have fewer workgroups than compute units: each then walks all of k alone, and the
// time of the launch is the time of one workgroup.  (BM = 256 -- half the dequantisation per matrix instruction, 256
// accumulator registers, one wave per SIMD -- measured no faster: 8192 rows of 14336 x 4096 856 against 822 us.)
constexpr int TK = 128, HK = 64;   // features per tile of the weights and per staged half of it
constexpr int AROW = HK + 8;                 // halves per activation row in LDS (the 16 rows of a 128-bit read pass in 16 distinct bank groups)

// KS > 1: KS (2, 4; 8 of one wave) such sets of waves share the workgroup's tile of C^T and split k between them (set kg takes tiles
// kg T / KS .. of every row, in LDS buffers of its own), and their accumulators are added through LDS at the end: for
// launches with so few workgroups that each compute unit would otherwise hold four waves that walk all of k alone.
// NW: waves per set (4; 2 or 1 -- 64 or 32 rows of the weights per workgroup -- when even the smallest tile above leaves
// compute units without a workgroup: the time of such a launch is the work of one compute unit).
template <int BM, int NI, int KS, int NW>
__global__ __launch_bounds__(64 * NW * KS, NW * KS >= 8 ? 1 : 2) void q4_0_tiled_matmul_kernel(MatMulDev p) {
    constexpr int MS = BM / 32;                  // 32-row subtiles of m
    constexpr int TS = 64 * NW;                  // threads of a set
    constexpr int TN = 32 * NI * NW;             // rows of the weights per workgroup
    // Half tiles of the activations on their way from memory: two where the registers allow it -- the small tiles exist
    // for launches in which a workgroup walks k alone, and a half tile's arithmetic is shorter than a trip to the L2.
    constexpr int PA = BM == 128 ? 1 : 2;
    // Tiles of the weights on their way from HBM, likewise: one tile's arithmetic of a small shape is about half of that trip.
    constexpr int PW = BM == 128 ? 1 : 3;
    constexpr int AP = BM * 8 / TS;              // 16-byte activation pieces per thread and half tile
    constexpr int RPP = TS / 8;                  // activation rows that the set's threads stage in one pass
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];   // [KS][2][BM AROW] halves; then the sums

    const int tid = threadIdx.x % TS, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) % NW), kg = __builtin_amdgcn_readfirstlane(threadIdx.x / TS);
    const int hb = lane >> 5, l32 = lane & 31;
    const int n0 = blockIdx.x * TN, m0 = blockIdx.y * BM, b = blockIdx.z, wb = b / p.ratio;
    const int groups = p.n / 16, T = p.k / TK;
    const int Tg = T / KS, tile0 = kg * Tg;      // this set's tiles of k: tile0 .. tile0 + Tg - 1 (the launcher: T % KS == 0)
    _Float16 *lds_a = reinterpret_cast<_Float16 *>(lds_raw) + kg * 2 * BM * AROW;

    // Both operands through buffer descriptors (one weight matrix and one batch of activations are below 4 GB: the
    // launcher checks): per-lane offsets are 32-bit and fixed, what moves along k is a scalar offset.  Activation rows
    // past m read as zeros: the range check sees the vector offset only, which is the piece's place in half tile 0 of
    // its row -- beyond the buffer exactly when the row is.
    // This lane's weight rows: n0 + 32 NI w + 32 i + l32, i.e. row l32 % 16 of row group n0 / 16 + 2 NI w + 2 i + l32 / 16
    // (groups past the end repeat the last one; their outputs are not stored).
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.codes + (int64_t)wb * groups * T * 1152), 0, (uint32_t)((int64_t)groups * T * 1152), 0x00020000);
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(p.act + (int64_t)b * p.m * p.k), 0, (uint32_t)((int64_t)p.m * p.k * 2), 0x00020000);
    uint32_t w_slot[NI], w_scale[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const uint32_t grp = (uint32_t)min(n0 / 16 + 2 * NI * w + 2 * i + (l32 >> 4), groups - 1);
        w_slot[i] = grp * (uint32_t)T * 1152u + 16 * (l32 & 15) + 256 * hb;
        w_scale[i] = grp * (uint32_t)T * 1152u + 1024 + 8 * (l32 & 15);
    }
    // activation piece j * TS + tid of a half tile: row RPP j + tid / 8 of the workgroup's BM, features 8 pc .. 8 pc + 7 of
    // the half (pc = tid % 8): features 8 pb .. 8 pb + 7 of its block pc / 4 (pb = pc % 4), which are halves pb / 2 of the
    // vectors g = 2 (pb % 2) and g + 1 of that block; vector 4 block + g of a row sits at 8 (4 block + g) halves
    const int a_row = tid >> 3, a_pc = tid & 7;
    uint32_t a_src[AP];   // bytes
#pragma unroll
    for (int j = 0; j < AP; j++) a_src[j] = (uint32_t)((m0 + RPP * j + a_row) * p.k + a_pc * 8) * 2;
    const int a_dst = a_row * AROW + (4 * (a_pc >> 2) + 2 * (a_pc & 1)) * 8 + 4 * ((a_pc >> 1) & 1);   // piece j: + RPP j AROW

    struct Weights { u32x4 c[NI][2]; u32x2 s[NI]; };   // a tile's slots g = hb, 2 + hb and scales, for each 32 rows of the wave
    u32x4 apre[PA][AP];
    auto prefetch_w = [&](Weights &wt, int t) {
#pragma unroll
        for (int i = 0; i < NI; i++) {
            wt.c[i][0] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_slot[i], (tile0 + t) * 1152, 0);
            wt.c[i][1] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_slot[i] + 512, (tile0 + t) * 1152, 0);
            wt.s[i] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, w_scale[i], (tile0 + t) * 1152, 0);
        }
    };
    auto prefetch_a = [&](int set, int it) {   // half tile `it` of this set's share of k
#pragma unroll
        for (int j = 0; j < AP; j++) apre[set][j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_src[j], (2 * tile0 + it) * HK * 2, 0);
    };
    auto stage_a = [&](int set, int buf) {
#pragma unroll
        for (int j = 0; j < AP; j++) {
            *reinterpret_cast<u32x2 *>(&lds_a[buf * BM * AROW + a_dst + RPP * j * AROW]) = u32x2{apre[set][j].x, apre[set][j].y};
            *reinterpret_cast<u32x2 *>(&lds_a[buf * BM * AROW + a_dst + RPP * j * AROW + 8]) = u32x2{apre[set][j].z, apre[set][j].w};   // vector g + 1
        }
    };

    float16_t acc[NI][MS];   // [n subtile][m subtile] of the wave's 32 NI x BM
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
        for (int j = 0; j < MS; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    Weights ring[PW];   // tiles t + 1 .. t + PW are on their way while a copy of tile t is used (sets that swap roles
                        // instead of the copy measured slower: 46.8 against 40.8 us for 128 rows of 14336 x 4096)
#pragma unroll
    for (int u = 0; u < PW; u++)
        if (u < Tg) prefetch_w(ring[u], u);
    prefetch_a(0, 0);
    stage_a(0, 0);
    if (PA == 2 && Tg * 2 > 1) prefetch_a(1, 1);
    const int a_frag = l32 * AROW + 8 * hb;
    auto tile = [&](int t, const Weights &wt, Weights &refill) {
        if (t + PW < Tg) prefetch_w(refill, t + PW);
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            // Half tile it = 2 t + hh of the activations is in buffer hh; every wave is done with the other buffer.  Half
            // it + PA is requested now (into the registers that held half it, PA = 2, or it + 1 just staged), and half
            // it + 1 is written into the other buffer after this half's arithmetic.
            __syncthreads();
            const bool more = 2 * t + hh + 1 < 2 * Tg;
            if (2 * t + hh + PA < 2 * Tg) prefetch_a(PA == 2 ? hh : 0, 2 * t + hh + PA);
            const _Float16 *at = &lds_a[hh * BM * AROW + a_frag];
            half8_t bf[2][MS];   // the activation fragments of a step are read during the step before
#pragma unroll
            for (int mm = 0; mm < MS; mm++) bf[0][mm] = *reinterpret_cast<const half8_t *>(at + 32 * mm * AROW);
#pragma unroll
            for (int step = 0; step < 4; step++) {   // block 2 hh + step / 2 of the tile, slots g = 2 (step % 2) + hb
                const int jj = step >> 1, st = step & 1, j = 2 * hh + jj;
                if (step + 1 < 4) {
#pragma unroll
                    for (int mm = 0; mm < MS; mm++) bf[(step + 1) & 1][mm] = *reinterpret_cast<const half8_t *>(at + 32 * mm * AROW + 16 * (step + 1));
                }
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const half2_t d2 = as_half2(perm(0u, wt.s[i][j >> 1], (j & 1) ? 0x03020302u : 0x01000100u));
                    const uint32_t word = wt.c[i][st][j];
                    uint32_t lo0, lo1, hi0, hi1;
                    dequant4(word & 0x0F0F0F0Fu, d2, lo0, lo1);
                    dequant4((word >> 4) & 0x0F0F0F0Fu, d2, hi0, hi1);
                    const half8_t af = __builtin_bit_cast(half8_t, u32x4{lo0, lo1, hi0, hi1});
#pragma unroll
                    for (int mm = 0; mm < MS; mm++) acc[i][mm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf[step & 1][mm], acc[i][mm], 0, 0, 0);
                }
            }
            if (more) stage_a(PA == 2 ? hh ^ 1 : 0, hh ^ 1);
        }
    };
    for (int t0 = 0; t0 < Tg; t0 += PW) {
#pragma unroll
        for (int u = 0; u < PW; u++)
            if (t0 + u < Tg) {
                const Weights cur = ring[u];
                tile(t0 + u, cur, ring[u]);
            }
    }

    if constexpr (KS > 1) {
        // The sets' accumulators, added pairwise through LDS (over the activation buffers, which every wave has left):
        // the upper half of the sets writes, the lower half adds, until set 0 holds the sum.  [set][wave][register][lane].
        float *red = reinterpret_cast<float *>(lds_raw);
        constexpr int PER_WAVE = NI * MS * 16 * 64;
#pragma unroll
        for (int half = KS / 2; half >= 1; half >>= 1) {
            __syncthreads();
            if (kg >= half && kg < 2 * half) {
                float *dst = red + ((kg - half) * NW + w) * PER_WAVE + lane;
#pragma unroll
                for (int i = 0; i < NI; i++)
#pragma unroll
                    for (int mm = 0; mm < MS; mm++)
#pragma unroll
                        for (int r = 0; r < 16; r++) dst[((i * MS + mm) * 16 + r) * 64] = acc[i][mm][r];
            }
            __syncthreads();
            if (kg < half) {
                const float *src = red + (kg * NW + w) * PER_WAVE + lane;
#pragma unroll
                for (int i = 0; i < NI; i++)
#pragma unroll
                    for (int mm = 0; mm < MS; mm++)
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[i][mm][r] += src[((i * MS + mm) * 16 + r) * 64];
            }
        }
        if (kg != 0) return;
    }

    // C^T[n, m]: register r of a lane is n = 8 (r / 4) + 4 hb + r % 4 of the 32 x 32 tile, m = lane % 32
    _Float16 *out = p.out + (int64_t)b * p.m * p.n;
#pragma unroll
    for (int mm = 0; mm < MS; mm++) {
        const int mi = m0 + 32 * mm + l32;
        if (mi >= p.m) continue;
        _Float16 *orow = out + (int64_t)mi * p.n;
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                const int ni = n0 + 32 * NI * w + 32 * i + 8 * rq + 4 * hb;
                half4_t h4;
#pragma unroll
                for (int e = 0; e < 4; e++) h4[e] = (_Float16)acc[i][mm][4 * rq + e];
                if (ni < p.n) *reinterpret_cast<half4_t *>(orow + ni) = h4;   // (n is a multiple of 16)
            }
    }
}

}  // namespace

// 2 = not taken (the caller runs the rows in groups on the matrix-vector kernels): f32 activations (their products stay
// in f32 there), k that is not a whole number of 64-element chunks, misaligned operands, offsets beyond 32 bits.
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
    if (tiled) {
        // 32-bit byte offsets inside one weight matrix and one batch of activations (rows up to 128 past m are addressed)
        if (n % 16 || k % TK || (n / 16) * (k / TK) * 1152 >= (1ll << 32) || (m + 128) * k >= (1ll << 30)) return 2;
        // The largest tile of C^T per workgroup -- 256 (n) x 128 (m), 256 x 64, 128 x 64 -- that still gives three
        // quarters of the compute units a workgroup (128 x 128 never has more workgroups than 256 x 64); the smallest
        // when none does, and then (or with 256 x 64) k
        // split over 2 or 4 sets of waves inside the workgroup while the workgroups are fewer than the compute units
        // can hold of that size.
        static const int forced_bm = getenv("TROCM_Q4_MATMUL_BM") ? atoi(getenv("TROCM_Q4_MATMUL_BM")) : 0;   // (measurements)
        static const int forced_ni = getenv("TROCM_Q4_MATMUL_NI") ? atoi(getenv("TROCM_Q4_MATMUL_NI")) : 0;
        static const int forced_ks = getenv("TROCM_Q4_MATMUL_KS") ? atoi(getenv("TROCM_Q4_MATMUL_KS")) : 0;
        const int64_t cus = num_compute_units();
        // (up to 32 activation rows: 256 x 32, 128 x 32 -- half the matrix instructions of a tile of 64 rows)
        const int shapes64[3][2] = {{128, 2}, {64, 2}, {64, 1}}, shapes32[3][2] = {{32, 2}, {32, 2}, {32, 1}};
        const int (*shapes)[2] = m <= 32 ? shapes32 : shapes64;
        int bm = shapes[2][0], ni = 1;
        for (int c = 0; c < 3; c++) {
            const int64_t wgs = ((n + 128 * shapes[c][1] - 1) / (128 * shapes[c][1])) * ((m + shapes[c][0] - 1) / shapes[c][0]) * act_batch;
            if (wgs * 4 >= cus * 3) {
                bm = shapes[c][0], ni = shapes[c][1];
                break;
            }
        }
        if (forced_bm == 32 || forced_bm == 64 || forced_bm == 128) bm = forced_bm;
        if (forced_ni == 1 || forced_ni == 2) ni = forced_ni;
        if (bm == 128) ni = 2;
        const int64_t ty = (m + bm - 1) / bm;
        if (ty > 65535) return 2;
        // ... and when that smallest tile still leaves compute units idle, sets of 2 waves or 1 (64 or 32 rows of the
        // weights per workgroup)
        static const int forced_nw = getenv("TROCM_Q4_MATMUL_NW") ? atoi(getenv("TROCM_Q4_MATMUL_NW")) : 0;
        int nw = 4;
        if (bm <= 64 && ni == 1) {
            while (nw > 1 && ((n + 32 * nw - 1) / (32 * nw)) * ty * act_batch * 4 < cus * 3) nw /= 2;
            if (forced_nw == 1 || forced_nw == 2 || forced_nw == 4) nw = forced_nw;
        }
        const int64_t txw = (n + 32 * ni * nw - 1) / (32 * ni * nw);
        int ks = 1;
        if (bm <= 64) {
            const int64_t wgs = txw * ty * act_batch, tiles = k / TK;
            if (ni == 1 && nw == 1 && wgs <= cus * 2 && tiles % 8 == 0) ks = 8;      // (sets of one wave: 8 of them, two such workgroups per compute unit)
            else if (ni == 1 && wgs * nw <= cus * 4 && tiles % 4 == 0) ks = 4;       // (16 waves of 128 registers fill a compute unit)
            else if (wgs * nw <= 2 * cus * 4 && tiles % 2 == 0) ks = 2;
        }
        if (forced_ks == 1 || ((forced_ks == 2 || ((forced_ks == 4 || (forced_ks == 8 && nw == 1)) && ni == 1)) && bm <= 64 && (k / TK) % forced_ks == 0)) ks = forced_ks;
        const dim3 tgrid((unsigned)txw, (unsigned)ty, (unsigned)act_batch);
        const size_t lds_act = (size_t)ks * 2 * bm * AROW * sizeof(_Float16);
        const size_t lds_red = ks > 1 ? (size_t)(ks / 2) * nw * ni * (bm / 32) * 16 * 64 * sizeof(float) : 0;
        const size_t lds = lds_act > lds_red ? lds_act : lds_red;
        auto launch = [&](auto kernel) -> int {
            if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
                (void)hipGetLastError();
                return fail("q4_0_matmul (tiled weights): %zu bytes of LDS were refused", lds);
            }
            hipLaunchKernelGGL(kernel, tgrid, dim3(64 * nw * ks), lds, s, p);
            return 0;
        };
        auto launch_small = [&](auto bm_tag, auto nw_tag) -> int {   // 64 or 32 activation rows, 32 rows of the weights per wave
            constexpr int BMc = decltype(bm_tag)::value, NWc = decltype(nw_tag)::value;
            if constexpr (NWc == 1)
                if (ks == 8) return launch(q4_0_tiled_matmul_kernel<BMc, 1, 8, 1>);
            return ks == 4 ? launch(q4_0_tiled_matmul_kernel<BMc, 1, 4, NWc>) : ks == 2 ? launch(q4_0_tiled_matmul_kernel<BMc, 1, 2, NWc>)
                                                                                        : launch(q4_0_tiled_matmul_kernel<BMc, 1, 1, NWc>);
        };
        auto launch_bm = [&](auto bm_tag) -> int {
            constexpr int BMc = decltype(bm_tag)::value;
            if (ni == 2) return ks == 2 ? launch(q4_0_tiled_matmul_kernel<BMc, 2, 2, 4>) : launch(q4_0_tiled_matmul_kernel<BMc, 2, 1, 4>);
            return nw == 4 ? launch_small(bm_tag, std::integral_constant<int, 4>()) : nw == 2 ? launch_small(bm_tag, std::integral_constant<int, 2>())
                                                                                               : launch_small(bm_tag, std::integral_constant<int, 1>());
        };
        int rc;
        if (bm == 128) rc = launch(q4_0_tiled_matmul_kernel<128, 2, 1, 4>);
        else if (bm == 64) rc = launch_bm(std::integral_constant<int, 64>());
        else rc = launch_bm(std::integral_constant<int, 32>());
        if (rc) return rc;
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail("q4_0_matmul (tiled weights) launch failed: %s", hipGetErrorString(e));
        return 0;
    }
    // 128 x 128 tiles unless they are fewer than the compute units: then 128 (n) x 64 (m), twice as many workgroups
    const int64_t gx = (n + BN - 1) / BN;
    const bool half_m = gx * ((m + 127) / 128) * act_batch < num_compute_units() && m > 64;
    const int64_t gy = half_m ? (m + 63) / 64 : (m + 127) / 128;
    if (gy > 65535) return 2;
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)act_batch);
    if (half_m)
        hipLaunchKernelGGL((q4_0_matmul_kernel<64>), grid, dim3(kMmThreads), 0, s, p);
    else
        hipLaunchKernelGGL((q4_0_matmul_kernel<128>), grid, dim3(kMmThreads), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0_matmul launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace trocm
