// Pieces shared by the split-K decode kernels (plain and quantised KV): launch geometry,
// kernel parameters, DPP wave reductions and the split-merge kernel.
#pragma once
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include "common.h"

namespace trocm {

struct DecodeDev {
    const char *q;
    char *out;
    const char *k, *v;
    int64_t kv_stride_b, kv_stride_h, kv_stride_t;  // bytes
    int T;                                          // valid tokens
    int tiles_per_split, nsplit;
    int Hq, Hkv;
    // Query heads per kv head.  The kernels are instantiated for G = 1, 2, 4, 8; another group size runs
    // on the next larger one: the extra heads of a workgroup repeat its last real head and write nothing.
    int g_real;
    float scale_log2;
    float *part_o;   // [B*Hkv*nsplit][G*D]
    float *part_ml;  // [B*Hkv*nsplit][2*G]
    // quantised KV only: f16 scale planes, [B, Hkv, cap, D/32]
    const char *k_scales, *v_scales;
    int64_t sc_stride_b, sc_stride_h;  // bytes
    // fused append (plain formats): the step's new K/V rows, dense [B or n_seq, Hkv, 1, D]; NULL = none
    const char *k_new, *v_new;
    int new_pos;   // token index of the fused new token (T - 1 for a growing cache, the cursor of a ring buffer)
    // dense f16/f32 kernel: 1 = the splits of a sequence take groups of kWaves tiles round-robin
    // (concurrent workgroups then read neighbouring addresses), 0 = contiguous tile ranges
    int interleave;
    int xcd_skew;                 // period (in rounds of groups) of the rounds that odd splits leave to even ones; 0: none
    // != NULL: arrival counters (one int per (batch, kv head), zero between launches); the last
    // workgroup of a sequence-head to arrive merges the splits itself and no merge launch follows
    int *counters;
    // additive mask of the q/out dtype, [mask_b, mask_h, 1, T] (NULL = none); byte strides, 0 on a broadcast axis
    const char *mask;
    int64_t mask_stride_b, mask_stride_h;
    // affine u8 caches (decode_mfma_kivi_body): the Keys' per-channel scales, f32 [B * Hkv, D]; k_scales / v_scales then
    // point at the Values' per-token scale and lo planes, f32 [B, Hkv, cap_rows], sc_stride_* their byte strides
    const float *chan_scale;
    // fused append with RoPE (f16, 16-wide tiles): cos / sin rows of D halves, one per sequence rope_stride_b bytes apart
    const char *rope_cos, *rope_sin;
    int64_t rope_stride_b;
    // matrix-core kernels, 8-row records with at most 4 real heads, in-kernel merge of up to 8 splits: rows 4..7 are neither
    // combined, stored nor merged (TROCM_DECODE_LIVE_TRIM=0 keeps them)
    int live_trim;
};
inline int decode_live_trim() {
    static const int on = getenv("TROCM_DECODE_LIVE_TRIM") ? atoi(getenv("TROCM_DECODE_LIVE_TRIM")) : 1;
    return on;
}

// Ragged batches: one work item = a tile range of one sequence (device copies of the host plan).
struct RaggedItem {
    const char *k, *v;   // planes of the sequence (kv head 0): f16/f32 rows or block codes
    int64_t stride_h;    // bytes between kv heads
    const char *ks, *vs; // quantised formats: the f16 block-scale planes (NULL otherwise)
    int64_t sc_stride_h; // bytes between kv heads in them
    int T, tile_begin, tile_end;
    int seq, split, nsplit, slot0;
};
struct RaggedSeqSlots {
    int slot0, nsplit;
};

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kTile = 32;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float readlane_f(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}
// DPP controls: row_ror:n rotates within a row of 16 lanes; quad_perm[1,0,3,2] swaps neighbours.
constexpr int kRowRor1 = 0x121, kRowRor2 = 0x122, kRowRor4 = 0x124, kRowRor8 = 0x128, kSwapPairs = 0xB1;

__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_f<kRowRor8>(x));
    x = fmaxf(x, dpp_f<kRowRor4>(x));
    x = fmaxf(x, dpp_f<kRowRor2>(x));
    x = fmaxf(x, dpp_f<kRowRor1>(x));
    return fmaxf(fmaxf(readlane_f(x, 0), readlane_f(x, 16)), fmaxf(readlane_f(x, 32), readlane_f(x, 48)));
}
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_f<kRowRor8>(x);
    x += dpp_f<kRowRor4>(x);
    x += dpp_f<kRowRor2>(x);
    x += dpp_f<kRowRor1>(x);
    return (readlane_f(x, 0) + readlane_f(x, 16)) + (readlane_f(x, 32) + readlane_f(x, 48));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 16 bytes of K against 16 bytes of Q: 8 f16 products or 4 f32 products, f32 accumulate.
// Vector elements are copied into scalars before any bit cast.
__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

template <typename T>
__device__ __forceinline__ float dot16(u32x4 k, u32x4 q, float acc);
template <>
__device__ __forceinline__ float dot16<__half>(u32x4 k, u32x4 q, float acc) {
    uint32_t k0 = k.x, k1 = k.y, k2 = k.z, k3 = k.w;
    uint32_t q0 = q.x, q1 = q.y, q2 = q.z, q3 = q.w;
    acc = __builtin_amdgcn_fdot2(as_half2(k0), as_half2(q0), acc, false);
    acc = __builtin_amdgcn_fdot2(as_half2(k1), as_half2(q1), acc, false);
    acc = __builtin_amdgcn_fdot2(as_half2(k2), as_half2(q2), acc, false);
    acc = __builtin_amdgcn_fdot2(as_half2(k3), as_half2(q3), acc, false);
    return acc;
}
template <>
__device__ __forceinline__ float dot16<float>(u32x4 k, u32x4 q, float acc) {
    uint32_t k0 = k.x, k1 = k.y, k2 = k.z, k3 = k.w;
    uint32_t q0 = q.x, q1 = q.y, q2 = q.z, q3 = q.w;
    acc = fmaf(as_f32(k0), as_f32(q0), acc);
    acc = fmaf(as_f32(k1), as_f32(q1), acc);
    acc = fmaf(as_f32(k2), as_f32(q2), acc);
    acc = fmaf(as_f32(k3), as_f32(q3), acc);
    return acc;
}

// The slice of a V row owned by one lane in the PV phase: EPL = D/16 elements.
template <typename T, int EPL>
struct VSlice;
template <>
struct VSlice<__half, 8> { typedef half8_t type; };
template <>
struct VSlice<__half, 4> { typedef half4_t type; };
template <>
struct VSlice<float, 8> { typedef float8_t type; };
template <>
struct VSlice<float, 4> { typedef float4_t type; };

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ __half from_f32<__half>(float x) { return __float2half_rn(x); }
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }

// Merge the per-split partials (O, m, l) of ONE query head h of a (batch, kv head) and write its
// output row; called by a workgroup of D threads, one output element per thread.  Partial records
// `first`, `first + stride`, ... (`nsplit` of them).  The (m, l) pairs go through LDS once and the
// O loads of different splits are independent, so the chain is two memory latencies long however
// many splits there are (with one thread looping over splits and heads a B=1 merge took as long
// as the attention itself).
constexpr int kMergeChunk = 256;
constexpr int kTailMergeMax = 8;   // most splits the in-kernel (last workgroup) merge handles
template <typename T, int D, int G>
__device__ __forceinline__ void merge_head(const DecodeDev &p, int64_t first, int64_t stride, int nsplit, int h,
                                           T *out_row, int tid) {
    __shared__ float lds_m[kMergeChunk], lds_l[kMergeChunk];
    float m_run = -INFINITY, acc = 0.0f, ll = 0.0f;
    for (int base = 0; base < nsplit; base += kMergeChunk) {
        const int n = min(kMergeChunk, nsplit - base);
        if (base) __syncthreads();
        for (int sp = tid; sp < n; sp += D) {
            const float *ml = p.part_ml + (first + (int64_t)(base + sp) * stride) * (2 * G);
            lds_m[sp] = ml[h];
            lds_l[sp] = ml[G + h];
        }
        __syncthreads();
        float cm = -INFINITY;
        for (int sp = 0; sp < n; sp++) cm = fmaxf(cm, lds_m[sp]);
        const float m_new = fmaxf(m_run, cm);
        const float m_ref = m_new == -INFINITY ? 0.0f : m_new;   // every split masked out with -inf so far: weights 0, not NaN
        const float keep = fast_exp2(m_run - m_ref);   // 0 on the first chunk
        acc *= keep;
        ll *= keep;
        m_run = m_new;
        const float *po = p.part_o + (first + (int64_t)base * stride) * (G * D) + h * D + tid;
        const int64_t po_step = stride * (G * D);
#pragma unroll 8
        for (int sp = 0; sp < n; sp++) {
            const float f = fast_exp2(lds_m[sp] - m_ref);
            acc += po[sp * po_step] * f;
            ll += lds_l[sp] * f;
        }
    }
    out_row[tid] = from_f32<T>(ll > 0.0f ? acc / ll : 0.0f);   // a row masked out entirely with -inf: zeros
}

// In-kernel merge by the last workgroup of a (sequence, kv head) to arrive.  Every workgroup calls this
// after storing its partial record with agent-scope (write-through) stores: it waits for its stores,
// signals its arrival on `counter`, and the workgroup that arrives last reads all `nsplit` records
// (first, first + stride, ...; at most kTailMergeMax) with agent-scope loads and writes the G output
// rows at `out`.  All loads of all splits are issued before the first use: one memory latency, not
// one per split.  The counter is left at zero for the next launch.
// MAXS: the most splits this instantiation merges (nsplit <= MAXS).
// LIVE: how many of a record's G rows are read (the rows of real heads come first; the matrix-core kernels pad their
// groups, and with up to half the rows real they skip the rest).
template <typename T, int D, int G, int LIVE = G, int MAXS = kTailMergeMax>
__device__ __forceinline__ void tail_merge(const DecodeDev &p, int *counter, int nsplit, int64_t first, int64_t stride,
                                           T *out, int tid) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial stores have completed
    __syncthreads();                                     // ... and so have the whole workgroup's
    __shared__ int s_last;
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = arrived == nsplit - 1;
        if (s_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    auto aload = [](const float *a) { return __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    constexpr int NE = (LIVE * D + kThreads - 1) / kThreads;
    float mv[NE][MAXS], lv[NE][MAXS], ov[NE][MAXS];
    const int64_t ml_step = stride * (2 * G), po_step = stride * (G * D);
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const int idx = min(tid + e * kThreads, G * D - 1);
        const int h = idx / D;
        const float *ml = p.part_ml + first * (2 * G) + h;
        const float *po = p.part_o + first * (G * D) + idx;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            const int spc = min(sp, nsplit - 1);   // splits past the last repeat it and get weight 0 below
            mv[e][sp] = aload(ml + spc * ml_step);
            lv[e][sp] = aload(ml + spc * ml_step + G);
            ov[e][sp] = aload(po + spc * po_step);
        }
    }
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const int idx = tid + e * kThreads;
        float mm = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) mm = fmaxf(mm, mv[e][sp]);
        if (mm == -INFINITY) mm = 0.0f;   // a row masked out entirely with -inf: weights 0, not NaN
        float acc = 0.0f, ll = 0.0f;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            const float f = sp < nsplit ? fast_exp2(mv[e][sp] - mm) : 0.0f;
            acc += ov[e][sp] * f;
            ll += lv[e][sp] * f;
        }
        if (idx < p.g_real * D) out[idx] = from_f32<T>(ll > 0.0f ? acc / ll : 0.0f);
    }
}

// tail_merge with two consecutive elements per thread: 64-bit agent-scope loads, half the instructions, and for 4 live
// rows of 128 one element pair per thread.  The records must have been stored the same way (two floats at a time).
template <typename T, int D, int G, int LIVE, int MAXS>
__device__ __forceinline__ void tail_merge_pairs(const DecodeDev &p, int *counter, int nsplit, int64_t first, int64_t stride,
                                                 T *out, int tid) {
    static_assert(D % 2 == 0, "pairs of elements of one row");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial stores have completed
    __syncthreads();                                     // ... and so have the whole workgroup's
    __shared__ int s_last_pairs;
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last_pairs = arrived == nsplit - 1;
        if (s_last_pairs) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last_pairs) return;
    auto aload = [](const float *a) { return __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    auto aload2 = [](const float *a) {
        return __hip_atomic_load(reinterpret_cast<const uint64_t *>(a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    constexpr int NE = (LIVE * D + 2 * kThreads - 1) / (2 * kThreads);
    float mv[NE][MAXS], lv[NE][MAXS];
    uint64_t ov[NE][MAXS];
    const int64_t ml_step = stride * (2 * G), po_step = stride * (G * D);
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const int idx = min(2 * (tid + e * kThreads), LIVE * D - 2);
        const int h = idx / D;
        const float *ml = p.part_ml + first * (2 * G) + h;
        const float *po = p.part_o + first * (G * D) + idx;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            const int spc = min(sp, nsplit - 1);   // splits past the last repeat it and get weight 0 below
            mv[e][sp] = aload(ml + spc * ml_step);
            lv[e][sp] = aload(ml + spc * ml_step + G);
            ov[e][sp] = aload2(po + spc * po_step);
        }
    }
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const int idx = 2 * (tid + e * kThreads);
        float mm = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) mm = fmaxf(mm, mv[e][sp]);
        if (mm == -INFINITY) mm = 0.0f;   // a row masked out entirely with -inf: weights 0, not NaN
        float acc0 = 0.0f, acc1 = 0.0f, ll = 0.0f;
#pragma unroll
        for (int sp = 0; sp < MAXS; sp++) {
            const float f = sp < nsplit ? fast_exp2(mv[e][sp] - mm) : 0.0f;
            acc0 += __builtin_bit_cast(float, (uint32_t)ov[e][sp]) * f;
            acc1 += __builtin_bit_cast(float, (uint32_t)(ov[e][sp] >> 32)) * f;
            ll += lv[e][sp] * f;
        }
        if (idx < p.g_real * D && idx < LIVE * D) {
            out[idx] = from_f32<T>(ll > 0.0f ? acc0 / ll : 0.0f);
            out[idx + 1] = from_f32<T>(ll > 0.0f ? acc1 / ll : 0.0f);
        }
    }
}

// The same for up to kWideMergeMax splits (small batches: 32 splits at batch 1), with G * kWideMergeMax <=
// kThreads: thread (h, sp) loads the (m, l) record of head h in split sp and the 32 threads of a head reduce
// them to weights, which go through `lds_w` (G * kWideMergeMax floats of LDS that nothing else uses any more);
// the outputs of all splits are requested before that, so the whole merge is one round trip to the L2 where
// a merge launch costs a launch gap and a kernel.
constexpr int kWideMergeMax = 32;
template <typename T, int D, int G>
__device__ __forceinline__ void tail_merge_wide(const DecodeDev &p, int *counter, int nsplit, int64_t first, int64_t stride,
                                                T *out, int tid, float *lds_w) {
    static_assert(G * kWideMergeMax <= kThreads, "one thread per (head, split)");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial stores have completed
    __syncthreads();                                     // ... and so have the whole workgroup's
    __shared__ int s_last_wide;
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last_wide = arrived == nsplit - 1;
        if (s_last_wide) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last_wide) return;
    auto aload = [](const float *a) { return __hip_atomic_load(a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    constexpr int NE = (G * D + kThreads - 1) / kThreads;
    const int64_t ml_step = stride * (2 * G), po_step = stride * (G * D);
    float ov[NE][kWideMergeMax];
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const float *po = p.part_o + first * (G * D) + min(tid + e * kThreads, G * D - 1);
#pragma unroll
        for (int sp = 0; sp < kWideMergeMax; sp++) ov[e][sp] = aload(po + min(sp, nsplit - 1) * po_step);
    }
    if (tid < G * kWideMergeMax) {
        const int h = tid / kWideMergeMax, sp = tid % kWideMergeMax;
        const float *ml = p.part_ml + first * (2 * G) + min(sp, nsplit - 1) * ml_step + h;
        const float m = aload(ml), l = aload(ml + G);
        float mm = m;
#pragma unroll
        for (int d = 1; d < kWideMergeMax; d <<= 1) mm = fmaxf(mm, __shfl_xor(mm, d, 64));
        const float f = sp < nsplit ? fast_exp2(m - (mm == -INFINITY ? 0.0f : mm)) : 0.0f;
        float ll = l * f;
#pragma unroll
        for (int d = 1; d < kWideMergeMax; d <<= 1) ll += __shfl_xor(ll, d, 64);
        lds_w[tid] = ll > 0.0f ? f / ll : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const int idx = tid + e * kThreads;
        const float *wh = lds_w + min(idx / D, G - 1) * kWideMergeMax;
        float acc = 0.0f;
#pragma unroll
        for (int sp = 0; sp < kWideMergeMax; sp++) acc += ov[e][sp] * wh[sp];
        if (idx < p.g_real * D) out[idx] = from_f32<T>(acc);
    }
}

// Merge launch: grid (kv_heads, batch, real query heads per kv head), D threads; runs after the split
// kernel on the same stream.
template <typename T, int D, int G>
__global__ __launch_bounds__(D) void sdpa_decode_merge_kernel(DecodeDev p) {
    const int kvh = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const int64_t bh = (int64_t)b * p.Hkv + kvh;
    T *out = reinterpret_cast<T *>(p.out) + ((int64_t)b * p.Hq + (int64_t)kvh * p.g_real + h) * D;
    merge_head<T, D, G>(p, bh * p.nsplit, 1, p.nsplit, h, out, threadIdx.x);
}

// Merge launch of the ragged batch: grid (kv_heads, sequences, G), D threads.
template <typename T, int D, int G>
__global__ __launch_bounds__(D) void sdpa_decode_ragged_merge_kernel(DecodeDev p, const RaggedSeqSlots *__restrict__ seqs) {
    const int kvh = blockIdx.x, seq = blockIdx.y, h = blockIdx.z;
    const RaggedSeqSlots ss = seqs[seq];
    if (ss.nsplit <= 1) return;
    T *out = reinterpret_cast<T *>(p.out) + ((int64_t)seq * p.Hq + (int64_t)kvh * p.g_real + h) * D;
    merge_head<T, D, G>(p, (int64_t)ss.slot0 * p.Hkv + kvh, p.Hkv, ss.nsplit, h, out, threadIdx.x);
}

}  // namespace

// The MFMA formulation of the ragged launch (sdpa_decode_mfma.hip); gp = its padded group size (8, 16, 32),
// which is also the stride of the partial records.
int decode_mfma_group(int64_t g_real);   // 0: not taken by the MFMA formulation
int launch_sdpa_decode_quant_mfma(DecodeDev &p, int kv_fmt, int64_t B, void *workspace, size_t workspace_bytes, hipStream_t s);
bool decode_quant_appends_in_kernel(int64_t g_real, float scale);
bool decode_quant_rotates_in_kernel(int64_t g_real);
int launch_sdpa_decode_ragged_mfma(const DecodeDev &p, int kv_fmt, int gp, int64_t D, const RaggedItem *items, int n_items,
                                   const RaggedSeqSlots *seqs, int n_seq, bool any_split, hipStream_t s);

// Partials: at most kMaxSplitRows rows of (D + 2) floats per query head.
constexpr int64_t kMaxSplitRows = 32768;
int choose_decode_splits(int64_t BH, int64_t G, int n_tiles, int wg_per_cu);
// The splits that the caller's workspace has room for (records of BH x splits x G rows of D + 2 floats behind the
// counter area), at least one: a call with a small or no workspace runs with fewer splits, it does not fail.
inline int fit_decode_splits(int nsplit, int64_t BH, int64_t G, int64_t D, const void *workspace, size_t workspace_bytes) {
    if (nsplit <= 1 || workspace == nullptr || workspace_bytes <= kWsCounterBytes) return 1;
    const int64_t per_split = BH * G * (D + 2) * (int64_t)sizeof(float);
    const int64_t fit = (int64_t)(workspace_bytes - kWsCounterBytes) / per_split;
    return (int)(fit < 1 ? 1 : fit < nsplit ? fit : nsplit);
}

}  // namespace trocm
