// Q4_0 weights in tiles of 16 rows x 128 features, and their products with a few activation rows: gfx950.
//
//   out[b, i, j] = sum_k act[b, i, k] * dequant(W[b / ratio, j, k])
//
// the matrix-vector arm of GgmlGemm (cuda/src/kernels/matmul/mod.rs:575-627) for weights whose row count is a
// multiple of 16 and whose row length is a multiple of 128: the matrices of a decoder.
//
// Layout.  The weights are constant, so they are laid out once, at load time, in the order in which the matrix
// instruction consumes them.  Tile (G, t) = rows 16 G .. 16 G + 15, features 128 t .. 128 t + 127 (4 blocks per row)
// is one record of 1152 bytes, the records of a row group consecutive in t:
//   bytes [0, 1024): slot l = r + 16 g (r = row in the group, g = 0..3) holds 16 bytes: word j = code bytes
//                    4 g .. 4 g + 3 of block 4 t + j of the row, i.e. its elements 4 g .. 4 g + 3 (low nibbles) and
//                    16 + 4 g .. 16 + 4 g + 3 (high nibbles) -- what lane l feeds v_mfma_f32_16x16x32_f16 as the B
//                    operand of block j;
//   bytes [1024, 1152): the f16 scales [r][j].
// A wave's loads are then one 128-bit and one 64-bit load per lane and tile, from nine consecutive cache lines of
// which every byte is used: a load instruction costs the compute unit's address path one step per cache line it
// touches, and rows of the [n, k/2] code plane put every lane group of a load on 16 different lines.
// trocm_q4_0_weights_export undoes the layout: the canonical 18-byte blocks come back unchanged.
//
// f16 activations, 1..16 rows (q4_0_tiled_mfma_kernel): KS waves share the tiles of a row group (wave q takes
// tiles q, q + KS, ...), a workgroup of 8 waves holds 8 / KS row groups behind one staged copy of the activations and
// walks `rounds` such sets.  Every wave keeps a ring of PD tiles in flight that runs on across the end of a round into
// the next round's first tiles, so that neither the reduction over the KS waves nor the barrier in front of it leaves
// the memory pipe idle.  Arithmetic: the contraction of the instruction is 32 deep, one quantisation block; the codes
// enter as the exact f16 numbers 64 + code (one v_perm_b32 per two codes, no subtraction), a second instruction per
// block with the constant operand -72 takes the offset off, both accumulate in f32 inside the instructions from zero,
// and the block's sum is scaled by its f16 scale with one fma per output.  Every product is exact; the sums round at
// the magnitude 72 |x| (1e-5 of a block's sum, below the f16 result's own rounding).
//
// f32 activations, 1..8 rows: the same kernel with v_mfma_f32_16x16x32_bf16.  Staging splits every activation into
// three bf16 numbers of 8 significant bits each (x = b1 + b2 + b3 exactly, by truncation and exact remainders), which
// become ROWS 4 i, 4 i + 1, 4 i + 2 of the instruction's A operand for activation row i of a set of four: one
// instruction forms the three partial products of four rows, each summed in f32 over all of k, and a lane's first
// three outputs are added at the end, smallest part first.  The codes enter as 16 + code, exact in bf16, so every
// product is exact: the arithmetic of an f32 kernel, over the whole range of f32, for the matrix instructions and LDS
// reads of an f16 row (rows 5..8: a second set, twice those).
//
// Roofline: HBM-bound on the weights: 18 bytes per 32 weights, read once.
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include <type_traits>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTile = 1152;        // bytes per tile record
constexpr int kTileScales = 1024;  // offset of the scales in a record
constexpr int kW = 8;              // waves per workgroup of the f16 kernel
constexpr int kActF16 = 0, kActF32Rows = 1, kActF32Rows2 = 2;   // how the activations enter the matrix instruction (see the kernel)

// ---- layout ---------------------------------------------------------------------------------------------------------
// Canonical blocks [rows, nb, 18 bytes] (f16 scale, 16 code bytes; 2-byte aligned) <-> tiles.  One thread per block.
__global__ __launch_bounds__(256) void q4_0_tiled_import_kernel(const uint16_t *__restrict__ src, uint8_t *__restrict__ tiles,
                                                                int64_t rows, int64_t nb) {
    const int64_t total = rows * nb, T = nb / 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t blk = idx % nb, row = idx / nb;
        const int r = (int)(row % 16), j = (int)(blk % 4);
        uint8_t *rec = tiles + ((row / 16) * T + blk / 4) * kTile;
        const uint16_t *i16 = src + idx * 9;
        *reinterpret_cast<uint16_t *>(rec + kTileScales + (r * 4 + j) * 2) = i16[0];
#pragma unroll
        for (int g = 0; g < 4; g++)
            *reinterpret_cast<uint32_t *>(rec + 16 * (r + 16 * g) + 4 * j) = (uint32_t)i16[1 + 2 * g] | ((uint32_t)i16[2 + 2 * g] << 16);
    }
}

__global__ __launch_bounds__(256) void q4_0_tiled_export_kernel(const uint8_t *__restrict__ tiles, uint16_t *__restrict__ dst,
                                                                int64_t rows, int64_t nb) {
    const int64_t total = rows * nb, T = nb / 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t blk = idx % nb, row = idx / nb;
        const int r = (int)(row % 16), j = (int)(blk % 4);
        const uint8_t *rec = tiles + ((row / 16) * T + blk / 4) * kTile;
        uint16_t *o = dst + idx * 9;
        o[0] = *reinterpret_cast<const uint16_t *>(rec + kTileScales + (r * 4 + j) * 2);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t w = *reinterpret_cast<const uint32_t *>(rec + 16 * (r + 16 * g) + 4 * j);
            o[1 + 2 * g] = (uint16_t)w, o[2 + 2 * g] = (uint16_t)(w >> 16);
        }
    }
}

// ---- products ---------------------------------------------------------------------------------------------------------
struct TiledDev {
    const uint8_t *tiles;     // [w_batch, n / 16, k / 128] records
    const void *act;          // [act_batch, m, k]
    void *out;                // [act_batch, m, n]
    int64_t act_stride_b, out_stride_b;   // elements between consecutive batches of act and out
    int n, k, m, ratio;       // ratio = act_batch / w_batch
    int T, groups;            // tiles per row group (k / 128), row groups per weight matrix (n / 16)
    int cq, nch;              // tiles per staged chunk of the activations, chunks (1: staged once per workgroup)
    int rounds;               // sets of row groups a workgroup walks
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// The four bytes of `c` hold codes (low nibbles) e..e+3 and (high nibbles) 16+e..16+e+3 of a block: the eight
// values 64 + code as f16, in that order.  0x5400 is the half 64, whose last place between 64 and 128 is 1/16: a
// code in the high nibble of the low byte adds exactly the code.  The 72 too many per weight come off in a second
// matrix instruction (its B operand the constant -72): 7 vector instructions per 8 weights instead of 11.
__device__ __forceinline__ half8_t codes_plus_64(uint32_t c) {
    const uint32_t lo = (c << 4) & 0xF0F0F0F0u, hi = c & 0xF0F0F0F0u;
    const uint32_t a = perm(0x54545454u, lo, 0x04010400u), b = perm(0x54545454u, lo, 0x04030402u);
    const uint32_t c2 = perm(0x54545454u, hi, 0x04010400u), d = perm(0x54545454u, hi, 0x04030402u);
    return __builtin_bit_cast(half8_t, u32x4{a, b, c2, d});
}

// As bf16 the offset can be smaller (the sums then round at a third of the magnitude): 0x4180 is 16, whose last place
// between 16 and 32 is 1/8: the code shifted left by three stays inside the low byte.  16 + code, and -24 in the
// second instruction.
__device__ __forceinline__ bf16x8_t codes_plus_16_bf16(uint32_t c) {
    const uint32_t lo = ((c << 3) & 0x78787878u) | 0x80808080u, hi = ((c >> 1) & 0x78787878u) | 0x80808080u;
    const uint32_t a = perm(0x41414141u, lo, 0x04010400u), b = perm(0x41414141u, lo, 0x04030402u);
    const uint32_t c2 = perm(0x41414141u, hi, 0x04010400u), d = perm(0x41414141u, hi, 0x04030402u);
    return __builtin_bit_cast(bf16x8_t, u32x4{a, b, c2, d});
}

// CHUNKED: the activations do not fit LDS and are staged in nch chunks per round.  (A kernel of its own: with loads
// for the staging inside the loop over the rounds, the compiler drains every load at the head of the tile loop.)
// ACT: kActF16 = f16 activations and output (up to 16 rows); kActF32Rows = f32 activations and output, up to 4 rows
// as three-part rows; kActF32Rows2 = 5..8 rows as two sets of them.
template <int KS, int PD, bool CHUNKED, int ACT>
__global__ __launch_bounds__(64 * kW, ACT == kActF32Rows2 ? 2 : 4) void q4_0_tiled_mfma_kernel(TiledDev p) {
    constexpr bool F32 = ACT != kActF16;
    constexpr int NSET = ACT == kActF32Rows2 ? 2 : 1;   // sets of four activation rows, an instruction per block each
    using ActT = typename std::conditional<F32, float, _Float16>::type;
    constexpr int LR = F32 ? 3 : 1;                  // rows of 16-bit numbers in LDS per activation row
    constexpr int kThreads = 64 * kW, S = kW / KS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int kc = p.cq * 128;                       // staged features per activation row
    uint16_t *lds_x = reinterpret_cast<uint16_t *>(lds_raw);                                // [m][kc] ([3 m][kc]: row 3 i + part), 16-byte vectors swizzled
    float *red = reinterpret_cast<float *>(lds_raw + (size_t)LR * p.m * kc * 2);            // [2][kW][4][64] (KS > 1)
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = w % KS, st = w / KS;               // this wave's share of a row group's tiles, its row group of the set
    const int b = blockIdx.y, wb = b / p.ratio;
    const ActT *act = reinterpret_cast<const ActT *>(p.act) + (int64_t)b * p.act_stride_b;
    ActT *out = reinterpret_cast<ActT *>(p.out) + (int64_t)b * p.out_stride_b;
    // output rows m..15 of the instruction (rows 4 i + 3 and 4 m.. of the three-part rows) are never stored: any row serves
    const int arow = F32 ? min(3 * (r16 >> 2) + min(r16 & 3, 2), 3 * p.m - 1) : min(r16, p.m - 1);
    const int arow2 = min(arow + 12, 3 * p.m - 1);   // (three-part rows: the second set of four rows)
    const int ni = p.T > q ? (p.T - q + KS - 1) / KS : 0;   // this wave's tiles of a row group: q + KS tt, tt < ni
    const int cqw = p.cq / KS;                       // ... of which a full chunk holds cqw (a multiple of PD when nch > 1)
    const uint8_t *wbase = p.tiles + (int64_t)wb * p.groups * p.T * kTile;
    const uint32_t lane_codes = 16 * lane, lane_scales = 8 * r16;

    // Slot d of the ring holds tile tt = d (mod PD) of some round.  The tiles are read through a buffer descriptor
    // per row group (base = the group's first record, size = its T records): a load past the group's end -- a wave's
    // share that is not a multiple of PD, a round that does not exist -- is still issued, returns zeros and moves no
    // data, so that no load sits behind a branch (which would turn every later wait for one load into a wait for all).
    u32x4 cn[PD];
    u32x2 sn[PD];
    const uint32_t m72 = F32 ? 0xC1C0C1C0u : 0xD480D480u;      // -24 as two bf16, -72 as two f16
    const u32x4 minus_72 = {m72, m72, m72, m72};                 // (the offset that the second instruction takes off)
    struct Group { const uint8_t *base; uint32_t bytes; };
    auto group_of = [&](int round) {
        const int64_t gi = (blockIdx.x + (int64_t)round * gridDim.x) * S + st;
        const bool valid = round < p.rounds && gi < p.groups;
        return Group{wbase + (valid ? gi : 0) * p.T * kTile, valid ? (uint32_t)p.T * kTile : 0u};
    };
    auto rsrc_of = [&](const Group &grp) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(grp.base), 0, grp.bytes, 0x00020000); };
    auto fetch = [&](int d, __amdgpu_buffer_rsrc_t rsrc, int tt) {
        const uint32_t rec = (uint32_t)(q + KS * tt) * kTile;       // tt >= ni: past the end
        cn[d] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, rec + lane_codes, 0, 0);
        sn[d] = __builtin_amdgcn_raw_buffer_load_b64(rsrc, rec + kTileScales + lane_scales, 0, 0);
    };

    // Chunk c of the activations: tiles c cq .. c cq + cq - 1 of every row, loaded 16 bytes (8 features) at a time, 8 (4)
    // loads of a thread in flight.  A tile's 16 vectors of 16 bytes are XOR-swizzled by the row, and features
    // 4 pb .. 4 pb + 3 of a block go to vector pb % 4, half pb / 4 of it, so that vector e of a block holds features
    // 4e..4e+3 and 16+4e..16+4e+3: the A operand of lane group e.  Every workgroup of the launch reads the same bytes:
    // each starts at another place of the chunk, so that at any moment the compute units ask different channels of the L2.
    constexpr int NP = CHUNKED ? 4 : 8;   // (registers)
    constexpr int PPT = F32 ? 32 : 16;    // 16-byte pieces of the source per tile and row: 4 f32 or 8 f16 features each
    // PRIVATE (every wave has tiles of its own, activations staged whole): a wave stages exactly the tiles it will read,
    // all rows of them, and nobody waits for anybody -- no barrier between the staging and the first tile.
    constexpr bool PRIVATE = KS == kW && !CHUNKED;
    auto stage = [&](int c, auto &&after_last_loads) {
        const int ntl = PRIVATE ? ni : min(p.cq, p.T - c * p.cq), per_row = ntl * PPT, total = p.m * per_row;
        constexpr int NTH = PRIVATE ? 64 : kThreads;   // threads that share the pieces
        if (total == 0) {
            after_last_loads();
            return;
        }
        const int start = (int)(((int64_t)blockIdx.x * 37 % 64) * total / 64);
        const uint32_t inv_per_row = 0xFFFFFFFFu / (uint32_t)per_row + 1;   // v / per_row = high word of v * this (v * per_row < 2^32)
        for (int base = 0; base < total; base += NTH * NP) {   // (uniform: every thread runs every pass)
            const int v0 = base + (PRIVATE ? lane : tid);
            u32x4 x[NP];
            // piece v: row i, tile tl of the chunk, piece pp of the tile (computed twice rather than kept)
            auto where = [&](int u, int &i, int &tl, int &pp) {
                int v = min(v0 + u * NTH, total - 1) + start;      // (past the end: the last piece again, not stored)
                if (v >= total) v -= total;
                i = (int)__umulhi((uint32_t)v, inv_per_row);
                const int rem = v - i * per_row;
                tl = rem / PPT, pp = rem % PPT;
                if constexpr (PRIVATE) tl = q + KS * tl;                 // (the wave's tl-th tile)
            };
#pragma unroll
            for (int u = 0; u < NP; u++) {
                int i, tl, pp;
                where(u, i, tl, pp);
                x[u] = *reinterpret_cast<const u32x4 *>(act + (int64_t)i * p.k + (int64_t)(c * p.cq + tl) * 128 + pp * (F32 ? 4 : 8));
            }
            if (base + NTH * NP >= total) after_last_loads();
#pragma unroll
            for (int u = 0; u < NP; u++) {
                if (v0 + u * NTH < total) {
                    int i, tl, pp;
                    where(u, i, tl, pp);
                    if constexpr (F32) {
                        // features 4 pp .. 4 pp + 3 of the tile: vector (pp / 8) * 4 + pp % 4, half (pp / 4) % 2 of it, in each of the row's three
                        const int vecg = (pp >> 3) * 4 + (pp & 3), hi = (pp >> 2) & 1;
                        const int in_row = tl * 128 + hi * 4;
                        // (the elements by name: indexed by the counter of an unrolled loop, this compiler has been seen
                        // to read element 0 of an ext-vector every time)
                        const uint32_t xe[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
                        uint32_t part[3][4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float x0 = __builtin_bit_cast(float, xe[e]);
                            part[0][e] = xe[e] & 0xFFFF0000u;                                     // the first 8 bits of x
                            const float r1 = x0 - __builtin_bit_cast(float, part[0][e]);          // exact
                            part[1][e] = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
                            const float r2 = r1 - __builtin_bit_cast(float, part[1][e]);          // exact, at most 8 bits left
                            part[2][e] = __builtin_bit_cast(uint32_t, r2);
                        }
#pragma unroll
                        for (int pl = 0; pl < 3; pl++)
                            *reinterpret_cast<u32x2 *>(lds_x + (3 * i + pl) * kc + in_row + (vecg ^ ((3 * i + pl) & 15)) * 8) =
                                u32x2{perm(part[pl][1], part[pl][0], 0x07060302u), perm(part[pl][3], part[pl][2], 0x07060302u)};
                    } else {
                        // features 8 pp .. 8 pp + 7 of the tile: the halves of two neighbouring vectors
                        const int vecg = (pp >> 2) * 4 + ((2 * pp) & 3), hi = (pp >> 1) & 1;
                        const int dst = i * kc + tl * 128 + hi * 4 + (vecg ^ (i & 15)) * 8;
                        *reinterpret_cast<u32x2 *>(lds_x + dst) = u32x2{x[u][0], x[u][1]};
                        *reinterpret_cast<u32x2 *>(lds_x + (dst ^ 8)) = u32x2{x[u][2], x[u][3]};   // vector vecg + 1 (vecg is even)
                    }
                }
            }
        }
    };

    // The ring's first two tiles, the activations, the rest of the ring: loads return in order, and what waits for
    // the activations must not wait for the whole ring (by then half of a small matrix).
    Group g_cur = group_of(0);
    const __amdgpu_buffer_rsrc_t rs0 = rsrc_of(g_cur);
    fetch(0, rs0, 0);
    fetch(1, rs0, 1);
    auto rest_of_ring = [&]() {
#pragma unroll
        for (int d = 2; d < PD; d++) fetch(d, rs0, d);
    };
    if constexpr (!CHUNKED) {
        stage(0, rest_of_ring);
        if constexpr (!PRIVATE) __syncthreads();
    } else {
        rest_of_ring();
    }

    for (int round = 0; round < p.rounds; round++) {
        const int64_t unit = blockIdx.x + (int64_t)round * gridDim.x;
        const bool gvalid = unit * S + st < p.groups;
        const int64_t gi = unit * S + st;
        const Group g_next = group_of(round + 1);
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f}, acc2 = {0.0f, 0.0f, 0.0f, 0.0f};

        for (int c = 0; c < (CHUNKED ? p.nch : 1); c++) {
            if constexpr (CHUNKED) {
                if (c || round) __syncthreads();   // the previous chunk has been read
                stage(c, []() {});
                __syncthreads();
            }
            const int tt0 = CHUNKED ? c * cqw : 0, tt_end = CHUNKED ? min(ni, tt0 + cqw) : ni;
            const int tl_off = q - c * p.cq;                      // tile tt of the wave sits at tl_off + KS tt of the chunk
            for (int l0 = tt0; l0 < tt_end; l0 += PD) {
                const bool more_here = l0 + PD < ni;              // the round has another batch (maybe in the next chunk)
                const __amdgpu_buffer_rsrc_t rs = rsrc_of(more_here ? g_cur : g_next);
#pragma unroll
                for (int d = 0; d < PD; d++) {
                    const int tt = l0 + d;
                    if (tt < ni) {                                // (a share that is not a multiple of PD: zeros were loaded)
                        // The four blocks side by side: reads, then the instructions that need only the activations,
                        // then those that need the codes.  (Reading a tile's activations during the tile before it
                        // measured slower: 9.4 against 8.9 us for one row of 14336 x 4096.)
                        const int tl = tl_off + KS * tt;
                        u32x4 a[4];
                        float4_t part[4];
                        if constexpr (F32) {
                            bf16x8_t codes[4];
#pragma unroll
                            for (int j = 0; j < 4; j++) codes[j] = codes_plus_16_bf16(cn[d][j]);
                            if constexpr (NSET == 2) {   // rows 4..7 first: their sums go to acc2 before part[] is reused
                                float4_t part2[4];
#pragma unroll
                                for (int j = 0; j < 4; j++) a[j] = *reinterpret_cast<const u32x4 *>(lds_x + arow2 * kc + (tl * 16 + ((j * 4 + g) ^ (arow2 & 15))) * 8);
#pragma unroll
                                for (int j = 0; j < 4; j++) part2[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[j]), __builtin_bit_cast(bf16x8_t, minus_72), float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                                for (int j = 0; j < 4; j++) part2[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[j]), codes[j], part2[j], 0, 0, 0);
#pragma unroll
                                for (int j = 0; j < 4; j++) {
                                    const float dsc = (float)__builtin_bit_cast(_Float16, (uint16_t)(sn[d][j >> 1] >> (16 * (j & 1))));
#pragma unroll
                                    for (int e = 0; e < 4; e++) acc2[e] = __builtin_fmaf(dsc, part2[j][e], acc2[e]);
                                }
                            }
#pragma unroll
                            for (int j = 0; j < 4; j++) a[j] = *reinterpret_cast<const u32x4 *>(lds_x + arow * kc + (tl * 16 + ((j * 4 + g) ^ arow)) * 8);
#pragma unroll
                            for (int j = 0; j < 4; j++) part[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[j]), __builtin_bit_cast(bf16x8_t, minus_72), float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                            for (int j = 0; j < 4; j++) part[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[j]), codes[j], part[j], 0, 0, 0);
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; j++) a[j] = *reinterpret_cast<const u32x4 *>(lds_x + arow * kc + (tl * 16 + ((j * 4 + g) ^ arow)) * 8);
#pragma unroll
                            for (int j = 0; j < 4; j++) part[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a[j]), __builtin_bit_cast(half8_t, minus_72), float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                            for (int j = 0; j < 4; j++) part[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a[j]), codes_plus_64(cn[d][j]), part[j], 0, 0, 0);
                        }
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float dsc = (float)__builtin_bit_cast(_Float16, (uint16_t)(sn[d][j >> 1] >> (16 * (j & 1))));
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[e] = __builtin_fmaf(dsc, part[j][e], acc[e]);
                        }
                    }
                    // The slot is refilled once its tile has been used, into the same registers, and the refills stay
                    // where they are written (moved to the top of the batch, the ring would need a second set).
                    asm volatile("" ::: "memory");
                    fetch(d, rs, more_here ? tt + PD : d);
                }
            }
        }
        g_cur = g_next;

        // acc[e] = partial out[4 g + e][16 gi + r16] (three-part rows: part e of out[g][16 gi + r16], smallest part first)
        const int64_t row = gi * 16 + r16;
        if constexpr (F32) {
            const float mine[2] = {(acc[2] + acc[1]) + acc[0], (acc2[2] + acc2[1]) + acc2[0]};
            if constexpr (KS == 1) {
#pragma unroll
                for (int z = 0; z < NSET; z++)
                    if (gvalid && 4 * z + g < p.m) out[(int64_t)(4 * z + g) * p.n + row] = mine[z];
            } else {
                float *rb = red + (round & 1) * (kW * 4 * 64);
#pragma unroll
                for (int z = 0; z < NSET; z++) rb[(w * 4 + z) * 64 + lane] = mine[z];
                __syncthreads();
                if (q < NSET) {   // (KS >= 2 here: wave 0 of the row group sums the first set, wave 1 the second)
                    float sum = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < KS; ww++) sum += rb[((st * KS + ww) * 4 + q) * 64 + lane];
                    if (gvalid && 4 * q + g < p.m) out[(int64_t)(4 * q + g) * p.n + row] = sum;
                }
            }
        } else if constexpr (KS == 1) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (gvalid && 4 * g + e < p.m) out[(int64_t)(4 * g + e) * p.n + row] = (ActT)acc[e];
        } else {
            // Two buffers by the round's parity: the barrier of the next round separates this round's reads from the
            // writes of the round after it.
            float *rb = red + (round & 1) * (kW * 4 * 64);
#pragma unroll
            for (int e = 0; e < 4; e++) rb[(w * 4 + e) * 64 + lane] = acc[e];
            __syncthreads();
#pragma unroll
            for (int e0 = 0; e0 < 4; e0 += KS) {
                const int e = e0 + q;
                if (e < 4) {
                    float sum = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < KS; ww++) sum += rb[((st * KS + ww) * 4 + e) * 64 + lane];
                    if (gvalid && 4 * g + e < p.m) out[(int64_t)(4 * g + e) * p.n + row] = (ActT)sum;
                }
            }
        }
        // Loads and stores share one counter and are not ordered against each other: with a store outstanding the
        // compiler makes every wait for a tile a wait for all memory traffic, and it places its waits for every path
        // at once.  So the path that has stored waits here, once per round, for its stores (and the next round's
        // first tiles): what enters the tile loop has only loads outstanding, and the ring's waits count tiles.
        if (round + 1 < p.rounds) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    }
}

int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return v ? atoi(v) : dflt;
}

template <int KS, int PD, bool CHUNKED, int ACT>
int launch_mfma_ks(TiledDev p, int64_t act_batch, int per_cu_forced, hipStream_t s) {
    constexpr int S = kW / KS;
    constexpr bool F32 = ACT != kActF16;
    const size_t lds = (size_t)p.m * p.cq * 128 * 2 * (F32 ? 3 : 1) + (KS > 1 ? (size_t)2 * kW * 4 * 64 * sizeof(float) : 0);
    if (lds > 64 * 1024 &&      // beyond the default limit of dynamic LDS: allowed per kernel (and device) on request
        hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_0_tiled_mfma_kernel<KS, PD, CHUNKED, ACT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return fail("q4_0_matvec (tiled weights): %zu bytes of LDS were refused", lds);
    }
    int64_t per_cu = (160 * 1024) / (int64_t)lds;
    constexpr int kMaxPerCu = ACT == kActF32Rows2 ? 1 : 2;     // (by registers: 4 or 5 waves per SIMD; 2 or 3 with two sets of f32 rows)
    if (per_cu > kMaxPerCu) per_cu = kMaxPerCu;
    if (per_cu < 1) per_cu = 1;
    if (per_cu_forced > 0) per_cu = per_cu_forced;
    const int64_t units = (p.groups + S - 1) / S;
    int64_t resident = (int64_t)num_compute_units() * per_cu / act_batch;
    if (resident < 1) resident = 1;
    int64_t wgs = units, rounds = 1;
    if (units > resident) {
        rounds = (units + resident - 1) / resident;
        wgs = (units + rounds - 1) / rounds;
    }
    p.rounds = (int)rounds;
    hipLaunchKernelGGL((q4_0_tiled_mfma_kernel<KS, PD, CHUNKED, ACT>), dim3((unsigned)wgs, (unsigned)act_batch), dim3(64 * kW), lds, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0_matvec (tiled weights) launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <bool CHUNKED, int ACT>
int launch_mfma_cf(const TiledDev &p, int ks, int64_t act_batch, int per_cu_forced, hipStream_t s) {
    switch (ks) {
        case 1: return launch_mfma_ks<1, 8, CHUNKED, ACT>(p, act_batch, per_cu_forced, s);
        case 2: return launch_mfma_ks<2, 8, CHUNKED, ACT>(p, act_batch, per_cu_forced, s);
        case 4: return launch_mfma_ks<4, 8, CHUNKED, ACT>(p, act_batch, per_cu_forced, s);
        default: return launch_mfma_ks<8, 4, CHUNKED, ACT>(p, act_batch, per_cu_forced, s);
    }
}

int launch_tiled_mfma(TiledDev p, bool f32, int64_t act_batch, hipStream_t s) {
    static const int forced_ks = env_int("TROCM_Q4T_KS", 0);
    static const int forced_per_cu = env_int("TROCM_Q4T_WG_PER_CU", 0);
    static const int forced_lds_kb = env_int("TROCM_Q4T_LDS_KB", 0);
    const int64_t cus = num_compute_units();
    // The fewest waves per row group that still give (nearly) every compute unit a workgroup, each wave then walking
    // the longest stream of tiles: 128256 x 4096: 1; 14336 x 4096: 2 (224 workgroups; one row 8.9 us, 8 rows 10.0 us;
    // with 4: 9.3 / 10.7; with 8: 9.1 / 10.3); 4096 x 4096 and 4096 x 14336: 8.
    int ks = 8;
    for (int c = 1; c <= 8; c *= 2)
        if (((int64_t)p.groups * c + kW - 1) / kW * act_batch * 8 >= cus * 7) {
            ks = c;
            break;
        }
    if (p.m <= 2) ks = 8;   // (one or two rows: never slower, 14336 x 4096 8.9 against 9.2 us)
    while (ks > 1 && ks > p.T) ks /= 2;
    if (forced_ks == 1 || forced_ks == 2 || forced_ks == 4 || forced_ks == 8) ks = forced_ks;
    int pd = ks == 8 ? 4 : 8;
    // The activations whole in LDS if they fit beside the partial sums (2 bytes per feature; 6 as the three bf16 parts of
    // f32 activations); else in chunks of a multiple of KS PD tiles: 64 KB (two workgroups per compute unit cover each
    // other's staging), or 128 KB where 64 KB hold no such chunk.
    const int64_t red = ks > 1 ? 2 * kW * 4 * 64 * 4 : 0;
    const int64_t per_tile = (int64_t)p.m * 256 * (f32 ? 3 : 1);
    const int64_t lds_all = forced_lds_kb > 0 ? (int64_t)forced_lds_kb * 1024 : 160 * 1024;
    if (per_tile * p.T + red <= lds_all) {
        p.cq = p.T, p.nch = 1;
    } else {
        const int ks_wanted = ks;
        while (ks > 1 && (int64_t)ks * (ks == 8 ? 4 : 8) * per_tile > 128 * 1024) ks /= 2;   // (a chunk holds KS PD tiles at least)
        if (f32 && p.m > 4 && ks < ks_wanted) {
            // 6..8 f32 rows of many features: chunks that small hold too few tiles for the waves of a row group, and
            // with fewer waves per group the launch has too few workgroups (8 rows of 4096 x 14336: 47.8 us; as two
            // launches of four rows 2 x 17.6).  Activation rows are k apart, output rows n.
            TiledDev lo = p, hi = p;
            lo.m = 4, hi.m = p.m - 4;
            hi.act = (const float *)p.act + 4 * (int64_t)p.k, hi.out = (float *)p.out + 4 * (int64_t)p.n;
            const int rc = launch_tiled_mfma(lo, f32, act_batch, s);
            return rc ? rc : launch_tiled_mfma(hi, f32, act_batch, s);
        }
        pd = ks == 8 ? 4 : 8;
        const int64_t step = ks * pd;
        static const int forced_chunk_kb = env_int("TROCM_Q4T_CHUNK_KB", 0);
        const int64_t first = forced_chunk_kb > 0 ? (int64_t)forced_chunk_kb * 1024 : 64 * 1024;
        int64_t cq = first / per_tile / step * step;
        if (cq < step) cq = (128 * 1024) / per_tile / step * step;
        if (cq < step) return fail("q4_0_matvec (tiled weights): %d activation rows leave no room for a chunk", p.m);
        p.cq = (int)cq, p.nch = (int)((p.T + cq - 1) / cq);
    }
    if (p.nch > 1)
        return !f32 ? launch_mfma_cf<true, kActF16>(p, ks, act_batch, forced_per_cu, s)
             : p.m <= 4 ? launch_mfma_cf<true, kActF32Rows>(p, ks, act_batch, forced_per_cu, s)
                        : launch_mfma_cf<true, kActF32Rows2>(p, ks, act_batch, forced_per_cu, s);
    return !f32 ? launch_mfma_cf<false, kActF16>(p, ks, act_batch, forced_per_cu, s)
         : p.m <= 4 ? launch_mfma_cf<false, kActF32Rows>(p, ks, act_batch, forced_per_cu, s)
                    : launch_mfma_cf<false, kActF32Rows2>(p, ks, act_batch, forced_per_cu, s);
}

}  // namespace

bool q4_0_tiled_layout_fits(int64_t n, int64_t k) {
    return n % 16 == 0 && k % 128 == 0 && n >= 16 && k >= 128 && (k / 128) * kTile < (1ll << 31);   // (32-bit offsets within a row group)
}
size_t q4_0_tiled_bytes(int64_t rows, int64_t k) { return (size_t)(rows / 16) * (size_t)(k / 128) * kTile; }

int launch_q4_0_tiled_import(const void *blocks, void *tiles, int64_t rows, int64_t k, hipStream_t s) {
    const int64_t total = rows * (k / 32);
    if (total == 0) return 0;
    int64_t grid = (total + 255) / 256;
    if (grid > 65535 * 16) grid = 65535 * 16;
    hipLaunchKernelGGL(q4_0_tiled_import_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const uint16_t *)blocks, (uint8_t *)tiles, rows, k / 32);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0 weights (tiling) launch failed: %s", hipGetErrorString(e));
    return 0;
}

int launch_q4_0_tiled_export(const void *tiles, void *blocks, int64_t rows, int64_t k, hipStream_t s) {
    const int64_t total = rows * (k / 32);
    if (total == 0) return 0;
    int64_t grid = (total + 255) / 256;
    if (grid > 65535 * 16) grid = 65535 * 16;
    hipLaunchKernelGGL(q4_0_tiled_export_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t *)tiles, (uint16_t *)blocks, rows, k / 32);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4_0 weights (export of tiles) launch failed: %s", hipGetErrorString(e));
    return 0;
}

// Tiled weights x activations for any m: f16 rows in groups of up to 16 (more than 16 rows go to the matrix-matrix
// kernel first, which reads the same tiles, when it takes the call), f32 rows in groups of up to 8.
int launch_q4_0_tiled_matvec(const void *tiles, int64_t w_batch, int64_t n, int64_t k, const void *act, int act_dtype,
                             int64_t act_batch, int64_t m, void *out, hipStream_t s) {
    if (n >= (1ll << 30) || k >= (1ll << 30) || act_batch > 65535) return fail("q4_0_matvec: shape too large");
    // (a row group's records are addressed through one buffer descriptor: 32-bit offsets)
    if ((k / 128) * kTile >= (1ll << 31)) return fail("q4_0_matvec: rows of %lld features are too long for the tiled layout", (long long)k);
    // Up to 16 f16 rows take one pass through the kernel above, more go to the matrix-matrix kernel (us, two passes here |
    // one launch there with 32 activation rows per workgroup: 24 rows of 14336 x 4096 21.3 | 13.5, of 4096 x 4096
    // 12.9 | 10.0, of 1024 x 4096 12.4 | 8.9, of 4096 x 14336 35.5 | 32.3; 17 rows of the last 29.0 | 32.3).
    static const int matmul_from = env_int("TROCM_Q4_MATMUL_FROM", 17);
    if (act_dtype == TROCM_F16 && m >= matmul_from && m > 16) {
        const int rc = launch_q4_0_matmul(tiles, nullptr, w_batch, n, k, act, act_dtype, act_batch, m, out, s, 1);
        if (rc != 2) return rc;
    }
    const int64_t es = act_dtype == TROCM_F16 ? 2 : 4, step = act_dtype == TROCM_F16 ? 16 : 8;
    for (int64_t i0 = 0; i0 < m; i0 += step) {
        TiledDev p;
        memset(&p, 0, sizeof(p));
        p.tiles = (const uint8_t *)tiles;
        p.act = (const char *)act + i0 * k * es, p.out = (char *)out + i0 * n * es;
        p.act_stride_b = m * k, p.out_stride_b = m * n;
        p.n = (int)n, p.k = (int)k, p.m = (int)(m - i0 < step ? m - i0 : step), p.ratio = (int)(act_batch / w_batch);
        p.T = (int)(k / 128), p.groups = (int)(n / 16);
        const int rc = launch_tiled_mfma(p, act_dtype != TROCM_F16, act_batch, s);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace trocm
