// Split-K flash-decode attention for gfx950 (q_len == 1), GQA head sharing.
//
// Work decomposition
//   grid = (splits, kv_heads, batch); one 256-thread workgroup (4 wavefronts of 64)
//   owns a contiguous range of 32-token tiles of one (batch, kv head) and serves all G
//   query heads of that KV head from a single read of K and V.  Wave w takes tiles
//   w, w+4, ... of the range; every wave keeps its own online-softmax state.
//
// Per 32-token tile, per wave
//   K  : the 32 rows are fetched with coalesced 128-bit loads (consecutive lanes,
//        consecutive bytes), parked in registers while the previous tile is computed,
//        then stored to a wave-private LDS tile with a per-row rotation of the 16-byte
//        chunks so that the transposed read below is bank-conflict free.
//   QK : lanes 2t and 2t+1 read the two halves of row t from LDS and form the G dot
//        products of token t against the query vectors (broadcast reads from LDS); one
//        DPP exchange joins the halves, no other cross-lane traffic.
//   softmax: tile maximum per head by a DPP wave reduction; p = exp2(s - m) per lane.
//   PV : p goes through LDS; the wave regroups as 4 row groups x 16 lanes, lane j owning
//        head_dim/16 output columns; V rows come straight from HBM, coalesced, prefetched
//        one tile ahead.
//
// Combination
//   waves are merged through LDS; if the launch has several splits, each workgroup
//   stores its unnormalised (O, m, l) to the workspace and a second, tiny launch on the
//   same stream merges the splits of every (batch, kv head) and writes the output.  (A
//   single-launch "last workgroup merges" scheme needs device-scope release/acquire fences,
//   i.e. an L2 write-back and invalidate per workgroup on this multi-XCD part; measured, that
//   tripled the kernel time.)  Logits are kept in log2 units (scale * log2 e folded in).
//
// Roofline: HBM-bound.  Algorithmic bytes per launch = 2*B*Hkv*T*D*e (K and V once per KV
// head) + Q read + O write.
#include <algorithm>
#include "decode_common.h"

namespace trocm {
namespace {

// Rotation of the 16-byte chunks of LDS row t.  A 128-bit LDS read pass covers 16 lanes =
// 8 rows x 2 half rows; with this rotation they fall into 16 different 16-byte bank groups.
template <int CPR>
__device__ __forceinline__ int rot(int row) {
    return CPR == 8 ? (row >> 1) : row;
}

// What one workgroup has to do: a tile range of one (sequence, kv head), and where its result goes.
struct DecodeWork {
    const char *q;      // the G query rows of this kv head
    char *out;          // the G output rows
    const char *kbase, *vbase;
    const char *k_new, *v_new;  // fused append: the row of token new_pos is read from here and stored to the cache
    int new_pos;
    int T;              // valid tokens of the sequence (including a fused new token)
    int tile_begin, tile_end;
    int tile_step;      // distance between a wave's successive tiles (kWaves for a contiguous range)
    bool direct;        // single split: write the output rows; else store partials at `part`
    int64_t part;       // index of the partial record
    // in-kernel merge by the last workgroup to arrive (counter != NULL): the sequence-head's records
    // are part_first + s * part_stride, s < nsplit
    int *counter;
    int nsplit;
    int64_t part_first, part_stride;
    const char *mask;   // additive mask row of this kv head's first query head (NULL = none), token 0
    int64_t mask_stride_h;
};

template <typename T, int D, int G, bool MASK>
__device__ __forceinline__ void decode_body(const DecodeDev &p, const DecodeWork &wk) {
    constexpr int RB = D * sizeof(T);   // bytes of one K/V row: 128, 256 or 512
    constexpr int CPR = RB / 16;        // 16-byte chunks per row: 8, 16, 32
    constexpr int HC = CPR / 2;         // chunks per half row (one QK lane)
    constexpr int KL = kTile * CPR / 64;  // K loads per lane per tile
    constexpr int EPL = D / 16;         // output columns per lane in the PV phase
    constexpr int VI = kTile / 4;       // V rows per lane per tile
    typedef typename VSlice<T, EPL>::type vslice_t;
    static_assert(RB == 128 || RB == 256 || RB == 512, "unsupported row size");

    __shared__ u32x4 lds_k[kWaves][kTile * CPR];
    __shared__ u32x4 lds_q[G * CPR];
    __shared__ float lds_p[kWaves][kTile * G];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, and the compiler is told so: tile bases stay in scalar registers

    const char *kbase = wk.kbase, *vbase = wk.vbase;
    const int seq_T = wk.T;
    const int new_pos = wk.k_new ? wk.new_pos : -1;   // the token that comes from the step's input, if any
    // a tile takes the plain path when it is full and does not hold the new token
    auto plain_tile = [&](int t0) { return t0 + kTile <= seq_T && !(new_pos >= t0 && new_pos < t0 + kTile); };
    const int tile_begin = wk.tile_begin, tile_end = wk.tile_end, tile_step = wk.tile_step;
    const int last_tok = seq_T - 1;

    float m[G], l[G], o[G][EPL];
#pragma unroll
    for (int h = 0; h < G; h++) {
        m[h] = -INFINITY;
        l[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; e++) o[h][e] = 0.0f;
    }

    // K load j of a tile fetches 16-byte chunk (j*64 + lane) of the tile, i.e. row
    // (j*64+lane)/CPR, chunk (j*64+lane)%CPR: consecutive lanes, consecutive bytes.
    // LDS slot of (row, chunk c): row*CPR + ((c + rot(row)) mod CPR).
    // Addresses are a wave-uniform tile base plus per-lane 32-bit offsets that never change;
    // only the one partial tile at the end of the sequence clamps its rows to the last token.
    const int rg = lane >> 4, j16 = lane & 15;
    const int qk_row = lane >> 1, qk_half = lane & 1;
    const uint32_t stride_t = (uint32_t)p.kv_stride_t;
    uint32_t k_off[KL], k_slot[KL], v_off[VI];
#pragma unroll
    for (int j = 0; j < KL; j++) {
        int L = j * 64 + lane;
        int row = L / CPR, c = L % CPR;
        k_off[j] = (uint32_t)row * stride_t + (uint32_t)c * 16u;
        k_slot[j] = row * CPR + ((c + rot<CPR>(row)) & (CPR - 1));
    }
#pragma unroll
    for (int i = 0; i < VI; i++) v_off[i] = (uint32_t)(4 * i + rg) * stride_t + (uint32_t)j16 * (uint32_t)sizeof(vslice_t);

    u32x4 kreg[KL];
    vslice_t vreg[VI];
    // Additive mask values of this lane's token, one per query head, fetched one tile ahead, right after
    // the softmax that consumed the previous ones (so no second copy stays live across the QK phase: the
    // G=4 kernel has no register to spare, and a spill reload in the loop waits for vmcnt(0), i.e. for
    // every prefetch in flight).  Rows past the end read the last token's value; they are discarded
    // below.  The masked kernel is a separate instantiation and always issues G loads (a head stride
    // of 0 when the mask is shared), so that the compiler can count outstanding loads exactly.
    constexpr bool has_mask = MASK;
    T mreg[G];
#pragma unroll
    for (int h = 0; h < G; h++) mreg[h] = from_f32<T>(0.0f);
    auto issue_mask = [&](int tile) {
        // wave-uniform row bases plus one 32-bit lane offset
        const uint32_t moff = (uint32_t)min(tile * kTile + qk_row, last_tok) * (uint32_t)sizeof(T);
#pragma unroll
        for (int h = 0; h < G; h++) mreg[h] = *reinterpret_cast<const T *>(wk.mask + min(h, p.g_real - 1) * wk.mask_stride_h + moff);
    };
    auto issue_k = [&](int tile) {
        const int t0 = tile * kTile;
        const char *base = kbase + (int64_t)t0 * p.kv_stride_t;
        if (plain_tile(t0)) {
#pragma unroll
            // streaming (non-temporal) loads: K and V are read once per launch; keeping them out of the
            // caches' replacement order is worth 8-9 % of a launch (batch 8: 53.8 -> 49.9 us, batch 32: 189 -> 172 us)
            for (int j = 0; j < KL; j++) kreg[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + k_off[j]));
        } else {
            // the sequence's last tile and the tile of a fused new token: rows past the end repeat the
            // last token; the new token comes from the step's input
#pragma unroll
            for (int j = 0; j < KL; j++) {
                int L = j * 64 + lane;
                int row = min(L / CPR, last_tok - t0), c = L % CPR;
                const char *cache_ptr = base + (uint32_t)row * stride_t + (uint32_t)c * 16u;
                const bool is_new = t0 + row == new_pos;
                kreg[j] = *reinterpret_cast<const u32x4 *>(is_new ? wk.k_new + c * 16 : cache_ptr);
            }
        }
    };
    auto issue_v = [&](int tile) {
        const int t0 = tile * kTile;
        const char *base = vbase + (int64_t)t0 * p.kv_stride_t;
        if (plain_tile(t0)) {
#pragma unroll
            for (int i = 0; i < VI; i++) vreg[i] = __builtin_nontemporal_load(reinterpret_cast<const vslice_t *>(base + v_off[i]));
        } else {
#pragma unroll
            for (int i = 0; i < VI; i++) {
                int row = min(4 * i + rg, last_tok - t0);
                const char *cache_ptr = base + (uint32_t)row * stride_t + (uint32_t)j16 * (uint32_t)sizeof(vslice_t);
                const bool is_new = t0 + row == new_pos;
                vreg[i] = *reinterpret_cast<const vslice_t *>(is_new ? wk.v_new + j16 * (int)sizeof(vslice_t) : cache_ptr);
            }
        }
    };

    // A fused new token is stored to its place in the cache here, by the first wave of the sequence-head's first
    // workgroup, ahead of the tile loop: stored from inside the loop, the store shared the vector-memory counter with
    // the prefetches, and the waits the compiler sizes for the path with the fewest operations in flight made every tile
    // wait for its newest loads as well.
    if (new_pos >= 0 && w == 0 && tile_begin == 0 && lane < 2 * CPR) {
        const int c = lane % CPR;
        const char *src = (lane < CPR ? wk.k_new : wk.v_new) + c * 16;
        char *dst = const_cast<char *>(lane < CPR ? kbase : vbase) + (int64_t)new_pos * p.kv_stride_t + c * 16;
        *reinterpret_cast<u32x4 *>(dst) = *reinterpret_cast<const u32x4 *>(src);
    }

    int tile = tile_begin + w;
    if (tile < tile_end) {
        if constexpr (has_mask) issue_mask(tile);
        issue_k(tile);
        issue_v(tile);
    }
    // ---- stage the G query vectors of this KV head (the first tile's K and V are already in flight) ----
    {
        const u32x4 *qg = reinterpret_cast<const u32x4 *>(wk.q);
        for (int i = tid; i < G * CPR; i += kThreads) lds_q[i] = qg[min(i / CPR, p.g_real - 1) * CPR + i % CPR];
    }
    __syncthreads();
    const u32x4 *lds_krow = &lds_k[w][qk_row * CPR];
    const int qk_rot = rot<CPR>(qk_row) + qk_half * HC;

    for (; tile < tile_end; tile += tile_step) {
        const int t0 = tile * kTile;
        // 1. park the K tile in LDS (rotated chunks); its registers are then refilled
#pragma unroll
        for (int j = 0; j < KL; j++) lds_k[w][k_slot[j]] = kreg[j];
        const bool more = tile + tile_step < tile_end;
        if (more) issue_k(tile + tile_step);

        // 2. scores of token (t0 + qk_row): this lane covers chunks [qk_half*HC, +HC)
        float s[G];
#pragma unroll
        for (int h = 0; h < G; h++) s[h] = 0.0f;
#pragma unroll 2
        for (int cc = 0; cc < HC; cc++) {
            u32x4 kc = lds_krow[(cc + qk_rot) & (CPR - 1)];
#pragma unroll
            for (int h = 0; h < G; h++) s[h] = dot16<T>(kc, lds_q[h * CPR + qk_half * HC + cc], s[h]);
        }
        const bool valid = (t0 + qk_row) < seq_T;
        // 3. online softmax (wave-uniform running maximum per head)
        float pr[G];
#pragma unroll
        for (int h = 0; h < G; h++) {
            float full = s[h] + dpp_f<kSwapPairs>(s[h]);  // join the two half rows
            float sv = valid ? full * p.scale_log2 : -INFINITY;
            if constexpr (has_mask) sv = __builtin_fmaf((float)mreg[h], 1.4426950408889634f, sv);
            float m_new = fmaxf(m[h], wave_max(sv));
            // a tile whose every token is masked with -inf must leave the state untouched, not NaN
            const float m_ref = (has_mask && m_new == -INFINITY) ? 0.0f : m_new;
            float alpha = fast_exp2(m[h] - m_ref);
            pr[h] = fast_exp2(sv - m_ref);
            l[h] = l[h] * alpha + pr[h];  // both lanes of a pair add p: halved at the end
            m[h] = m_new;
#pragma unroll
            for (int e = 0; e < EPL; e++) o[h][e] *= alpha;
        }
        if constexpr (has_mask) {
            if (more) issue_mask(tile + tile_step);
        }
        if (qk_half == 0) {
            if constexpr (G == 4) {
                float4_t t4 = {pr[0], pr[1], pr[2], pr[3]};
                *reinterpret_cast<float4_t *>(&lds_p[w][qk_row * G]) = t4;
            } else {
#pragma unroll
                for (int h = 0; h < G; h++) lds_p[w][qk_row * G + h] = pr[h];
            }
        }
        // 4. O += P V (row group rg takes tokens 4*i + rg)
#pragma unroll
        for (int i = 0; i < VI; i++) {
            float pp[G];
            if constexpr (G == 4) {
                float4_t t4 = *reinterpret_cast<const float4_t *>(&lds_p[w][(4 * i + rg) * G]);
                pp[0] = t4[0], pp[1] = t4[1], pp[2] = t4[2], pp[3] = t4[3];
            } else {
#pragma unroll
                for (int h = 0; h < G; h++) pp[h] = lds_p[w][(4 * i + rg) * G + h];
            }
            vslice_t vv = vreg[i];
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                float vf = (float)vv[e];
#pragma unroll
                for (int h = 0; h < G; h++) o[h][e] = fmaf(pp[h], vf, o[h][e]);
            }
        }
        // 5. V of the wave's next tile (in flight while the next tile's QK runs)
        if (more) issue_v(tile + tile_step);
    }

    // ---- merge the 4 row groups of the wave, then the 4 waves through LDS ----------------
#pragma unroll
    for (int h = 0; h < G; h++) {
        l[h] = 0.5f * wave_sum(l[h]);
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            float x = o[h][e];
            x += __shfl_xor(x, 16, 64);
            x += __shfl_xor(x, 32, 64);
            o[h][e] = x;
        }
    }
    __syncthreads();  // every wave is done with its K tile: the space is reused below
    float *comb = reinterpret_cast<float *>(&lds_k[0][0]);  // [kWaves][G*D + 2*G]
    constexpr int kCombStride = G * D + 2 * G;
    static_assert(sizeof(float) * kWaves * kCombStride <= sizeof(u32x4) * kWaves * kTile * CPR, "combine buffer");
    if (rg == 0) {
#pragma unroll
        for (int h = 0; h < G; h++)
#pragma unroll
            for (int e = 0; e < EPL; e++) comb[w * kCombStride + h * D + j16 * EPL + e] = o[h][e];
    }
    if (lane == 0) {
#pragma unroll
        for (int h = 0; h < G; h++) {
            comb[w * kCombStride + G * D + h] = m[h];
            comb[w * kCombStride + G * D + G + h] = l[h];
        }
    }
    __syncthreads();

    T *out = reinterpret_cast<T *>(wk.out);
    for (int idx = tid; idx < G * D; idx += kThreads) {
        int h = idx / D;
        float mm = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) mm = fmaxf(mm, comb[ww * kCombStride + G * D + h]);
        // a range masked out entirely with -inf yields the neutral record (0, -inf, 0), not NaN
        const float mm_ref = mm == -INFINITY ? 0.0f : mm;
        float acc = 0.0f, ll = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
            float f = fast_exp2(comb[ww * kCombStride + G * D + h] - mm_ref);
            acc += comb[ww * kCombStride + idx] * f;
            ll += comb[ww * kCombStride + G * D + G + h] * f;
        }
        if (wk.direct) {
            if (h < p.g_real) out[idx] = from_f32<T>(ll > 0.0f ? acc / ll : 0.0f);
        } else if (wk.counter == nullptr) {
            int64_t slot = wk.part;
            p.part_o[slot * (G * D) + idx] = acc;
            if ((idx % D) == 0) {
                p.part_ml[slot * (2 * G) + h] = mm;
                p.part_ml[slot * (2 * G) + G + h] = ll;
            }
        } else {
            // Stores that are visible to every compute unit of the device when they complete (they
            // go through this XCD's L2): no cache write-back is needed before signalling arrival.
            int64_t slot = wk.part;
            __hip_atomic_store(&p.part_o[slot * (G * D) + idx], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((idx % D) == 0) {
                __hip_atomic_store(&p.part_ml[slot * (2 * G) + h], mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&p.part_ml[slot * (2 * G) + G + h], ll, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (wk.direct || wk.counter == nullptr) return;

    // ---- the last workgroup of this sequence-head to arrive merges the splits -------------------
    tail_merge<T, D, G>(p, wk.counter, wk.nsplit, wk.part_first, wk.part_stride, out, tid);
}

// Dense batch: grid (splits, kv_heads, batch); every sequence has the same length.
template <typename T, int D, int G, bool MASK>
__global__ __launch_bounds__(kThreads, (D * sizeof(T) <= 256 && G <= 4) ? 2 : 1) void sdpa_decode_kernel(DecodeDev p) {
    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    DecodeWork wk;
    const int64_t row = ((int64_t)b * p.Hq + (int64_t)kvh * p.g_real) * D * (int64_t)sizeof(T);
    wk.q = p.q + row;
    wk.out = p.out + row;
    wk.kbase = p.k + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    wk.vbase = p.v + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    const int64_t new_row = ((int64_t)b * p.Hkv + kvh) * D * (int64_t)sizeof(T);
    wk.k_new = p.k_new ? p.k_new + new_row : nullptr;
    wk.v_new = p.v_new ? p.v_new + new_row : nullptr;
    wk.T = p.T;
    wk.new_pos = p.new_pos;
    const int n_tiles = (p.T + kTile - 1) / kTile;
    if (p.interleave) {
        wk.tile_begin = split * kWaves;
        wk.tile_end = n_tiles;
        wk.tile_step = kWaves * p.nsplit;
    } else {
        wk.tile_begin = split * p.tiles_per_split;
        wk.tile_end = min(n_tiles, wk.tile_begin + p.tiles_per_split);
        wk.tile_step = kWaves;
    }
    wk.direct = p.nsplit == 1;
    const int64_t bh = (int64_t)b * p.Hkv + kvh;
    wk.part = bh * p.nsplit + split;
    wk.counter = p.counters ? p.counters + bh : nullptr;
    wk.nsplit = p.nsplit;
    wk.part_first = bh * p.nsplit;
    wk.part_stride = 1;
    wk.mask = MASK ? p.mask + (int64_t)b * p.mask_stride_b + (int64_t)kvh * p.g_real * p.mask_stride_h : nullptr;
    wk.mask_stride_h = p.mask_stride_h;
    decode_body<T, D, G, MASK>(p, wk);
}

// Ragged batch: grid (work items, kv_heads).  An item is a tile range of one sequence; the
// host cuts every sequence into ranges of about the same number of tiles, so that 64
// sequences whose lengths differ 64-fold still load all compute units evenly.
template <typename T, int D, int G>
__global__ __launch_bounds__(kThreads, (D * sizeof(T) <= 256 && G <= 4) ? 2 : 1) void sdpa_decode_ragged_kernel(
    DecodeDev p, const RaggedItem *__restrict__ items) {
    const RaggedItem it = items[blockIdx.x];
    const int kvh = blockIdx.y;
    DecodeWork wk;
    const int64_t row = ((int64_t)it.seq * p.Hq + (int64_t)kvh * p.g_real) * D * (int64_t)sizeof(T);
    wk.q = p.q + row;
    wk.out = p.out + row;
    wk.kbase = it.k + (int64_t)kvh * it.stride_h;
    wk.vbase = it.v + (int64_t)kvh * it.stride_h;
    const int64_t new_row = ((int64_t)it.seq * p.Hkv + kvh) * D * (int64_t)sizeof(T);
    wk.k_new = p.k_new ? p.k_new + new_row : nullptr;
    wk.v_new = p.v_new ? p.v_new + new_row : nullptr;
    wk.T = it.T;
    wk.new_pos = it.T - 1;
    wk.tile_begin = it.tile_begin;
    wk.tile_end = it.tile_end;
    wk.tile_step = kWaves;
    wk.direct = it.nsplit == 1;
    wk.part = ((int64_t)it.slot0 + it.split) * p.Hkv + kvh;
    wk.counter = nullptr;
    wk.nsplit = it.nsplit;
    wk.part_first = (int64_t)it.slot0 * p.Hkv + kvh;
    wk.part_stride = p.Hkv;
    wk.mask = nullptr;
    wk.mask_stride_h = 0;
    decode_body<T, D, G, false>(p, wk);
}

template <typename T, int D, int G>
void launch_both(const DecodeDev &p, dim3 grid, hipStream_t s) {
    if (p.mask)
        hipLaunchKernelGGL((sdpa_decode_kernel<T, D, G, true>), grid, dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL((sdpa_decode_kernel<T, D, G, false>), grid, dim3(kThreads), 0, s, p);
    if (p.nsplit > 1 && p.counters == nullptr)
        hipLaunchKernelGGL((sdpa_decode_merge_kernel<T, D, G>), dim3(grid.y, grid.z, p.g_real), dim3(D), 0, s, p);
}

template <typename T, int D>
int launch_g(const DecodeDev &p, int G, dim3 grid, hipStream_t s) {
    switch (G) {
        case 1: launch_both<T, D, 1>(p, grid, s); break;
        case 2: launch_both<T, D, 2>(p, grid, s); break;
        case 4: launch_both<T, D, 4>(p, grid, s); break;
        case 8: launch_both<T, D, 8>(p, grid, s); break;
        default: return 2;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_decode launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace

size_t decode_workspace_bytes(int64_t B, int64_t Hq, int64_t D) {
    int64_t rows = B * Hq > kMaxSplitRows ? B * Hq : kMaxSplitRows;
    return kWsCounterBytes + kWsPlanBytes + (size_t)rows * (size_t)(D + 2) * sizeof(float) + 256;
}

// Number of splits.  Measured on MI355X (8k context, f16, G=4): one workgroup per compute
// unit is the sweet spot -- each wave already keeps a 16 KiB tile in flight, so more
// workgroups add merge work and scheduling rounds without adding bandwidth (B=8: 4 splits
// = 256 workgroups 45.9 us; 8 splits 48.9 us; 32 splits 55.5 us).  Never fewer than one
// tile per wave, bounded by the workspace.  The quantised kernels are ALU/latency-limited and
// do better with two workgroups per compute unit (Q8_0, 16k context: 79.7 us vs 94.4 us).
int choose_decode_splits(int64_t BH, int64_t G, int n_tiles, int wg_per_cu) {
    static const int forced = getenv("TROCM_DECODE_SPLITS") ? atoi(getenv("TROCM_DECODE_SPLITS")) : 0;  // experiment knob, like tract's declare_knob!
    int64_t target = (int64_t)num_compute_units() * wg_per_cu;
    int64_t ns = forced > 0 ? forced : (target + BH / 2) / BH;
    int64_t max_by_tiles = (n_tiles + kWaves - 1) / kWaves;
    if (ns > max_by_tiles) ns = max_by_tiles;
    int64_t max_by_ws = kMaxSplitRows / (BH * G);
    if (ns > max_by_ws) ns = max_by_ws;
    if (ns < 1) ns = 1;
    if (forced <= 0) {   // no more splits than shorten the longest wave's run: the same critical path with fewer partial records
        const int64_t groups = max_by_tiles, longest = (groups + ns - 1) / ns;   // groups of kWaves tiles; groups per split
        ns = (groups + longest - 1) / longest;
    }
    return (int)ns;
}

int launch_sdpa_decode(const SdpaArgs &a, hipStream_t s) {
    if (a.Sq != 1) return 2;
    {   // grouped heads: the MFMA formulation (it declines f32 and masks over rows whose length is not a multiple of 4)
        const int rc = launch_sdpa_decode_mfma(a, s);
        if (rc != 2) return rc;
    }
    if (a.rope_cos) return 2;   // the rotation of q and k_new is built into the MFMA kernel only
    if (a.kv_fmt != TROCM_F16 && a.kv_fmt != TROCM_F32) return 2;
    if (a.q_dtype != a.kv_fmt) return 2;
    if (a.D != 64 && a.D != 128) return 2;
    if (a.Hq % a.Hkv) return 2;
    const int64_t g_real = a.Hq / a.Hkv;
    if (g_real > 8) return 2;
    const int64_t G = g_real <= 2 ? g_real : g_real <= 4 ? 4 : 8;   // the instantiation that runs it
    size_t es = elem_bytes(a.kv_fmt);
    // 128-bit loads: rows and bases must be 16-byte aligned
    if ((a.kv_stride_b * es) % 16 || (a.kv_stride_h * es) % 16 || (a.kv_stride_t * es) % 16) return 2;
    if ((uintptr_t)a.k % 16 || (uintptr_t)a.v % 16 || (uintptr_t)a.q % 16) return 2;
    if (a.Sk <= 0 || a.Sk > (1ll << 30)) return 2;
    int64_t BH = a.B * a.Hkv;
    if (BH > (int64_t)(kWsCounterBytes / sizeof(int)) || a.B > 65535 || a.Hkv > 65535) return 2;

    int n_tiles = (int)((a.Sk + kTile - 1) / kTile);
    int nsplit = fit_decode_splits(choose_decode_splits(BH, G, n_tiles, 1), BH, G, a.D, a.workspace, a.workspace_bytes);
    int tps = (n_tiles + nsplit - 1) / nsplit;
    nsplit = (n_tiles + tps - 1) / tps;  // no empty split
    DecodeDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const char *)a.q;
    p.out = (char *)a.out;
    p.k = (const char *)a.k;
    p.v = (const char *)a.v;
    p.kv_stride_b = a.kv_stride_b * es;
    p.kv_stride_h = a.kv_stride_h * es;
    p.kv_stride_t = a.kv_stride_t * es;
    p.T = (int)a.Sk;
    p.tiles_per_split = tps;
    p.nsplit = nsplit;
    // Round-robin groups of kWaves tiles over the splits of a sequence (measured 1-5 % faster than
    // contiguous ranges: concurrent workgroups read neighbouring addresses).  TROCM_DECODE_INTERLEAVE=0
    // restores contiguous ranges.
    static const int interleave = getenv("TROCM_DECODE_INTERLEAVE") ? atoi(getenv("TROCM_DECODE_INTERLEAVE")) : 1;
    p.interleave = interleave;
    p.Hq = (int)a.Hq;
    p.Hkv = (int)a.Hkv;
    p.g_real = (int)g_real;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    p.k_new = (const char *)a.k_new;
    p.v_new = (const char *)a.v_new;
    p.new_pos = a.new_pos >= 0 ? (int)a.new_pos : (int)a.Sk - 1;
    if (p.k_new && (p.v_new == nullptr || (uintptr_t)p.k_new % 16 || (uintptr_t)p.v_new % 16)) return 2;
    if (a.mask) {   // [mask_b, mask_h, 1, Sk] dense
        p.mask = (const char *)a.mask;
        p.mask_stride_h = a.mask_h > 1 ? a.Sk * (int64_t)es : 0;
        p.mask_stride_b = a.mask_b > 1 ? a.mask_h * a.Sk * (int64_t)es : 0;
    }
    p.part_ml = (float *)((char *)a.workspace + kWsCounterBytes);
    p.part_o = p.part_ml + (size_t)BH * nsplit * 2 * G;
    // With few splits the last workgroup of a (batch, kv head) to arrive merges them itself; with many
    // (small batches) the merge launch, which spreads the work over the chip, is faster (measured
    // B=1, 32 splits: 21 us against 14.5 us).  TROCM_DECODE_TAIL_MERGE=0 always uses the launch.
    static const int tail_merge = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    p.counters = (tail_merge && nsplit > 1 && nsplit <= kTailMergeMax) ? (int *)a.workspace : nullptr;
    dim3 grid(nsplit, (unsigned)a.Hkv, (unsigned)a.B);
    if (a.kv_fmt == TROCM_F16)
        return a.D == 128 ? launch_g<__half, 128>(p, (int)G, grid, s) : launch_g<__half, 64>(p, (int)G, grid, s);
    return a.D == 128 ? launch_g<float, 128>(p, (int)G, grid, s) : launch_g<float, 64>(p, (int)G, grid, s);
}

}  // namespace trocm

namespace trocm {
namespace {

// Pinned staging for the per-call plan of a ragged launch (a few KiB): a small ring per host
// thread, each slot guarded by an event so that a slot is not rewritten while its copy is
// still in flight.  A kernel copies the plan into the workspace: a copy command between two
// kernels of one stream hands the stream to a DMA engine and back, which left the device idle for
// 27..49 us per step (64 sequences, 16 KiB of plan); the copy kernel reads the pinned pages itself.
constexpr int kStageSlots = 4;
struct StageSlot {
    void *host = nullptr;
    void *host_dev = nullptr;   // the same pages as the device addresses them
    hipEvent_t done = nullptr;
    bool in_flight = false;
};

__global__ __launch_bounds__(256) void plan_upload_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int n16) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}
thread_local StageSlot g_stage[kStageSlots];
thread_local int g_stage_next = 0;

int acquire_stage(StageSlot **out) {
    StageSlot &sl = g_stage[g_stage_next];
    g_stage_next = (g_stage_next + 1) % kStageSlots;
    if (!sl.host) {
        TROCM_HIP(hipHostMalloc(&sl.host, kWsPlanBytes, hipHostMallocMapped));
        TROCM_HIP(hipHostGetDevicePointer(&sl.host_dev, sl.host, 0));
        TROCM_HIP(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
    } else if (sl.in_flight) {
        TROCM_HIP(hipEventSynchronize(sl.done));
    }
    sl.in_flight = false;
    *out = &sl;
    return 0;
}

}  // namespace

int upload_table(const void *src, size_t bytes, void *dst, hipStream_t s) {
    TROCM_REQUIRE(bytes <= kWsPlanBytes, "upload_table: %zu bytes exceed the staging slot", bytes);
    if (bytes == 0) return 0;
    StageSlot *stage;
    if (acquire_stage(&stage)) return 1;
    memcpy(stage->host, src, bytes);
    const int n16 = (int)((bytes + 15) / 16);
    hipLaunchKernelGGL(plan_upload_kernel, dim3((n16 + 255) / 256), dim3(256), 0, s, (const uint4 *)stage->host_dev, (uint4 *)dst, n16);
    TROCM_HIP(hipGetLastError());
    TROCM_HIP(hipEventRecord(stage->done, s));
    stage->in_flight = true;
    return 0;
}

namespace {

template <typename T, int D, int G>
void launch_ragged(const DecodeDev &p, const RaggedItem *items, int n_items, const RaggedSeqSlots *seqs, int n_seq,
                   bool any_split, hipStream_t s) {
    hipLaunchKernelGGL((sdpa_decode_ragged_kernel<T, D, G>), dim3(n_items, p.Hkv), dim3(kThreads), 0, s, p, items);
    if (any_split)
        hipLaunchKernelGGL((sdpa_decode_ragged_merge_kernel<T, D, G>), dim3(p.Hkv, n_seq, p.g_real), dim3(D), 0, s, p, seqs);
}

template <typename T, int D>
int launch_ragged_g(const DecodeDev &p, int G, const RaggedItem *items, int n_items, const RaggedSeqSlots *seqs,
                    int n_seq, bool any_split, hipStream_t s) {
    switch (G) {
        case 1: launch_ragged<T, D, 1>(p, items, n_items, seqs, n_seq, any_split, s); break;
        case 2: launch_ragged<T, D, 2>(p, items, n_items, seqs, n_seq, any_split, s); break;
        case 4: launch_ragged<T, D, 4>(p, items, n_items, seqs, n_seq, any_split, s); break;
        case 8: launch_ragged<T, D, 8>(p, items, n_items, seqs, n_seq, any_split, s); break;
        default: return 2;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("ragged sdpa_decode launch failed: %s", hipGetErrorString(e));
    return 0;
}

// One launch per sequence on the caller's stream: the fall-back for shapes and formats the
// ragged kernel does not cover (launches on one stream are ordered, so they share the workspace).
int ragged_per_sequence(const void *q, void *out, int q_dtype, int kv_fmt, int64_t n_seq, int64_t Hq, int64_t Hkv,
                        int64_t D, const RaggedSeq *seqs, float scale, void *workspace, size_t workspace_bytes,
                        hipStream_t s) {
    size_t es = elem_bytes(q_dtype);
    for (int64_t i = 0; i < n_seq; i++) {
        SdpaArgs a;
        memset(&a, 0, sizeof(a));
        a.q = (const char *)q + (size_t)i * Hq * D * es;
        a.out = (char *)out + (size_t)i * Hq * D * es;
        a.q_dtype = q_dtype, a.kv_fmt = kv_fmt;
        a.k = seqs[i].k, a.v = seqs[i].v, a.k_scales = seqs[i].k_scales, a.v_scales = seqs[i].v_scales;
        a.B = 1, a.Hq = Hq, a.Hkv = Hkv, a.Sq = 1, a.Sk = seqs[i].len, a.D = D;
        a.kv_stride_t = D, a.kv_stride_h = seqs[i].cap * D, a.kv_stride_b = Hkv * seqs[i].cap * D;
        a.mask_b = a.mask_h = 1;
        a.scale = scale;
        a.workspace = workspace, a.workspace_bytes = workspace_bytes;
        int rc = is_quant(kv_fmt) ? launch_sdpa_decode_quant(a, s) : launch_sdpa_decode(a, s);
        if (rc == 2) rc = launch_sdpa_generic(a, s);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace

// Ragged decode: one launch for all sequences.  The host cuts the sequences into work items
// of about equal tile counts, uploads the plan (items + per-sequence slot ranges) into the
// head of the workspace, and the kernels index it by blockIdx.
int launch_sdpa_decode_ragged(const void *q, void *out, int q_dtype, int kv_fmt, int64_t n_seq, int64_t Hq, int64_t Hkv,
                              int64_t D, const RaggedSeq *seqs, float scale, void *workspace, size_t workspace_bytes,
                              const void *k_new, const void *v_new, hipStream_t s, const void *rope_cos, const void *rope_sin) {
    const int64_t g_real = Hq / Hkv;
    // grouped heads over f16 or block-quantised caches: the MFMA formulation (sdpa_decode_mfma.hip)
    const bool quant = is_quant(kv_fmt);
    int mfma_gp = (kv_fmt == TROCM_F16 || (quant && q_dtype == TROCM_F16 && D == 128)) ? decode_mfma_group(g_real) : 0;
    // one head per kv head over quantised caches: the vector-ALU kernel has no ragged form, and one launch on the
    // matrix cores beats a launch per sequence
    if (quant && q_dtype == TROCM_F16 && D == 128 && g_real == 1) mfma_gp = 8;
    const int64_t G = mfma_gp ? mfma_gp : g_real <= 2 ? g_real : g_real <= 4 ? 4 : 8;   // the instantiation that runs it
    const int64_t rb = kv_fmt == TROCM_Q8_0 ? D : kv_fmt == TROCM_Q4_0 ? D / 2 : D * (int64_t)elem_bytes(kv_fmt);   // bytes per token row
    bool fast = quant ? mfma_gp != 0 && (k_new == nullptr || (g_real > 1 && decode_quant_appends_in_kernel(g_real, scale)))
                      : (kv_fmt == TROCM_F16 || kv_fmt == TROCM_F32) && q_dtype == kv_fmt && (D == 64 || D == 128) &&
                            g_real >= 1 && (g_real <= 8 || mfma_gp);
    fast = fast && workspace != nullptr && (uintptr_t)q % 16 == 0 && n_seq <= 2048 && Hkv <= 65535;
    for (int64_t i = 0; i < n_seq && fast; i++) {
        fast = (uintptr_t)seqs[i].k % 16 == 0 && (uintptr_t)seqs[i].v % 16 == 0 && seqs[i].len < (1ll << 30) &&
               (seqs[i].cap * rb) % 16 == 0;
        if (quant)
            fast = fast && seqs[i].k_scales && seqs[i].v_scales && (uintptr_t)seqs[i].k_scales % 4 == 0 &&
                   (uintptr_t)seqs[i].v_scales % 4 == 0;
    }
    if (k_new && ((uintptr_t)k_new % 16 || (uintptr_t)v_new % 16)) fast = false;
    if (rope_cos) {   // q and k_new rotated on the way in: the 16-wide f16 body, or the (head, block) bodies over quantised caches
        const bool covered = k_new && rope_sin && q_dtype == TROCM_F16 && mfma_gp != 0 && (uintptr_t)rope_cos % 16 == 0 &&
                             (uintptr_t)rope_sin % 16 == 0 && (D * 2) % 16 == 0 &&
                             (quant ? decode_quant_rotates_in_kernel(g_real) : kv_fmt == TROCM_F16 && mfma_gp <= 16);
        if (!covered) return 2;
    }
    if (!fast) {
        if (k_new) return 2;  // the caller appends explicitly, then calls again without a fused append
        return ragged_per_sequence(q, out, q_dtype, kv_fmt, n_seq, Hq, Hkv, D, seqs, scale, workspace, workspace_bytes, s);
    }

    // ---- plan ----------------------------------------------------------------------------------
    int64_t total_tiles = 0;
    for (int64_t i = 0; i < n_seq; i++) total_tiles += (seqs[i].len + kTile - 1) / kTile;
    TROCM_REQUIRE(workspace_bytes > kWsCounterBytes + kWsPlanBytes, "sdpa workspace too small for a ragged launch (%zu bytes)",
                  workspace_bytes);
    // Partial records are needed only by the items of sequences that are cut: a sequence that is one item writes its
    // output rows itself.  (Two limits, then: items in the plan table, records in the rest of the workspace.)
    const int64_t rows_cap = (int64_t)((workspace_bytes - kWsCounterBytes - kWsPlanBytes) / ((D + 2) * sizeof(float)));
    const int64_t max_slots_ws = rows_cap / (Hkv * G);  // a record has a row per (padded) query head of every kv head
    const int64_t max_items_tbl =
        ((int64_t)kWsPlanBytes - n_seq * (int64_t)sizeof(RaggedSeqSlots)) / (int64_t)sizeof(RaggedItem);
    TROCM_REQUIRE(max_items_tbl >= n_seq, "ragged decode: the plan area holds %lld work items, fewer than the %lld sequences",
                  (long long)max_items_tbl, (long long)n_seq);
    // Workgroups (items x kv heads) per compute unit: two are resident at a time, and the last round of
    // them is only partly full, so more and smaller items shorten the tail at the cost of partial records.
    static const int wg_per_cu = getenv("TROCM_RAGGED_WG_PER_CU") ? atoi(getenv("TROCM_RAGGED_WG_PER_CU")) : 0;
    int64_t want_items = wg_per_cu > 0 ? ((int64_t)num_compute_units() * wg_per_cu + Hkv - 1) / Hkv : num_compute_units();
    if (want_items < 1) want_items = 1;
    int64_t tiles_per_item = (total_tiles + want_items - 1) / want_items;
    if (tiles_per_item < kWaves) tiles_per_item = kWaves;
    int64_t n_items = 0, n_slots = 0;
    for (;;) {   // ends at the latest when no sequence is cut: n_seq items, no records
        n_items = n_slots = 0;
        for (int64_t i = 0; i < n_seq; i++) {
            int64_t tiles = (seqs[i].len + kTile - 1) / kTile;
            int64_t ns = (tiles + tiles_per_item - 1) / tiles_per_item;
            n_items += ns;
            if (ns > 1) n_slots += ns;
        }
        if (n_items <= max_items_tbl && n_slots <= max_slots_ws) break;
        tiles_per_item += (tiles_per_item + 3) / 4;
    }
    StageSlot *stage;
    if (acquire_stage(&stage)) return 1;
    RaggedItem *items = (RaggedItem *)stage->host;
    RaggedSeqSlots *slots = (RaggedSeqSlots *)(items + n_items);
    int64_t it = 0, slot_it = 0;
    bool any_split = false;
    int64_t max_split = 1;
    for (int64_t i = 0; i < n_seq; i++) {
        int64_t tiles = (seqs[i].len + kTile - 1) / kTile;
        int64_t ns = (tiles + tiles_per_item - 1) / tiles_per_item;
        int64_t tps = (tiles + ns - 1) / ns;
        ns = (tiles + tps - 1) / tps;
        slots[i].slot0 = (int)slot_it;   // first partial record of the sequence (unused when it is not cut)
        slots[i].nsplit = (int)ns;
        if (ns > 1) slot_it += ns;
        any_split |= ns > 1;
        if (ns > max_split) max_split = ns;
        for (int64_t sp = 0; sp < ns; sp++, it++) {
            RaggedItem &r = items[it];
            r.k = (const char *)seqs[i].k;
            r.v = (const char *)seqs[i].v;
            r.stride_h = seqs[i].cap * rb;
            r.ks = (const char *)seqs[i].k_scales, r.vs = (const char *)seqs[i].v_scales;
            r.sc_stride_h = seqs[i].cap * (D / 32) * 2;
            r.T = (int)seqs[i].len;
            r.tile_begin = (int)(sp * tps);
            r.tile_end = (int)((sp + 1) * tps < tiles ? (sp + 1) * tps : tiles);
            r.seq = (int)i, r.split = (int)sp, r.nsplit = (int)ns, r.slot0 = slots[i].slot0;
        }
    }
    n_items = it;
    // Longest items first: the workgroups that start last, when the device is no longer full, are the short ones.
    // (An item carries its own partial slot, so the order is free.)
    std::stable_sort(items, items + n_items, [](const RaggedItem &a, const RaggedItem &b) {
        return a.tile_end - a.tile_begin > b.tile_end - b.tile_begin;
    });
    // the seq table sits right after the items actually emitted
    RaggedSeqSlots *slots_packed = (RaggedSeqSlots *)(items + n_items);
    if (slots_packed != slots) memmove(slots_packed, slots, (size_t)n_seq * sizeof(RaggedSeqSlots));
    size_t plan_bytes = (size_t)n_items * sizeof(RaggedItem) + (size_t)n_seq * sizeof(RaggedSeqSlots);
    {
        const int n16 = (int)((plan_bytes + 15) / 16);   // the slot and the plan area are both kWsPlanBytes long
        hipLaunchKernelGGL(plan_upload_kernel, dim3((n16 + 255) / 256), dim3(256), 0, s, (const uint4 *)stage->host_dev,
                           (uint4 *)((char *)workspace + kWsCounterBytes), n16);
        TROCM_HIP(hipGetLastError());
    }
    TROCM_HIP(hipEventRecord(stage->done, s));
    stage->in_flight = true;

    DecodeDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const char *)q;
    p.out = (char *)out;
    p.kv_stride_t = rb;
    p.Hq = (int)Hq;
    p.Hkv = (int)Hkv;
    p.g_real = (int)g_real;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.k_new = (const char *)k_new;
    p.v_new = (const char *)v_new;
    if (rope_cos) p.rope_cos = (const char *)rope_cos, p.rope_sin = (const char *)rope_sin, p.rope_stride_b = D * 2;
    p.live_trim = decode_live_trim();
    p.part_ml = (float *)((char *)workspace + kWsCounterBytes + kWsPlanBytes);
    p.part_o = p.part_ml + (size_t)slot_it * Hkv * 2 * G;
    const RaggedItem *d_items = (const RaggedItem *)((char *)workspace + kWsCounterBytes);
    const RaggedSeqSlots *d_slots = (const RaggedSeqSlots *)(d_items + n_items);
    // The MFMA kernel merges the splits of a sequence-head itself when none has more than it can hold in registers.
    static const int tail = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    if (tail && mfma_gp && mfma_gp <= 8 && any_split && max_split <= kWideMergeMax &&
        n_seq * Hkv <= (int64_t)(kWsCounterBytes / sizeof(int)))
        p.counters = (int *)workspace;
    if (mfma_gp) return launch_sdpa_decode_ragged_mfma(p, kv_fmt, mfma_gp, D, d_items, (int)n_items, d_slots, (int)n_seq, any_split, s);
    if (kv_fmt == TROCM_F16)
        return D == 128 ? launch_ragged_g<__half, 128>(p, (int)G, d_items, (int)n_items, d_slots, (int)n_seq, any_split, s)
                        : launch_ragged_g<__half, 64>(p, (int)G, d_items, (int)n_items, d_slots, (int)n_seq, any_split, s);
    return D == 128 ? launch_ragged_g<float, 128>(p, (int)G, d_items, (int)n_items, d_slots, (int)n_seq, any_split, s)
                    : launch_ragged_g<float, 64>(p, (int)G, d_items, (int)n_items, d_slots, (int)n_seq, any_split, s);
}
}  // namespace trocm
