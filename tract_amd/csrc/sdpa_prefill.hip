// MFMA prefill attention for gfx950: q_len > 1, f16 in/out, f32 accumulate, causal
// (bottom-right aligned) or unmasked, GQA, K/V read in place from the capacity buffer.
//
// Formulation (transposed, so that every per-query softmax scalar lives in one lane):
//   S^T = K . Q^T      v_mfma_f32_32x32x16_f16, A = K rows (key-major, contraction over d),
//                      B = Q rows held in registers for the whole kernel
//   O^T = V^T . P^T    A = V^T fragments, B = P^T taken straight from the S^T accumulators
//                      (rounded to f16), contraction over keys
// In the 32x32 accumulator layout a lane holds ONE query column (lane % 32) and 16 of the 32
// rows (keys, or output features): row maxima and sums over keys are in-lane reductions plus
// one exchange between the two half-waves, and the rescaling factors of the online softmax
// apply to the lane's own O^T registers.
//
// A wave owns 32 queries and, per workgroup tile, 64 keys.  The waves of a workgroup are
// arranged WM x WN: WM query groups (BLOCK_M = 32*WM) times WN key slices (BLOCK_N = 64*WN);
// waves that share queries keep separate online-softmax states and are merged through LDS at
// the end.  2x2 (64 queries per workgroup) keeps more compute units busy when there are few
// query tiles, 4x2 (eight waves, 128 queries) halves the K/V staging per query when there are
// many.  This kernel serves prompts too short for sdpa_prefill_pp.hip, whose grouped-head
// workgroups are the fast path.
//
// K and V tiles: global -> registers (prefetched one tile ahead) -> LDS, both row-major with
// padded rows, written with 128-bit stores.  K fragments are plain 128-bit LDS reads.  For V
// the MFMA wants 8 KEYS per lane at a fixed feature while V rows are feature-major: the
// fragments are read with gfx950's transposing LDS load (ds_read_b64_tr_b16).  Measured
// semantics of that load: in each block of 16 lanes, lane i receives element i%4 of the four
// 8-byte rows addressed by lanes i/4, i/4+4, i/4+8, i/4+12.  So source lane s of a block points
// at V[key(s/4)][16 features of the block + 4*(s%4)] and lane i comes back with 4 keys of its
// own feature; two such loads give the 8 keys of one contraction step, in the order in which
// the S^T accumulator registers hold them (rows 4hb..4hb+3, then 8+4hb..8+4hb+3).
//
// Roofline: MFMA-bound.  FLOPs = 4 * B * Hq * D * (visible query-key pairs).
#include <hip/hip_fp16.h>
#include <string.h>
#include <stdlib.h>
#include "common.h"

namespace trocm {
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));


struct PrefillDev {
    const _Float16 *q;
    _Float16 *out;
    const _Float16 *k, *v;
    int64_t kv_stride_b, kv_stride_h, kv_stride_t;  // elements
    int B, Hq, Hkv, Sq, Sk;
    int causal;
    int n_qtiles;
    float scale_log2;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Transposing 64-bit LDS load of 16-bit elements (see the header comment for its lane mapping).
__device__ __forceinline__ half4_t lds_read_tr16(const _Float16 *lds_ptr) {
    typedef __attribute__((address_space(3))) short4_t *lds_v4_ptr;
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_ptr)(uintptr_t)(uint32_t)(uintptr_t)lds_ptr);
    return __builtin_bit_cast(half4_t, r);
}

template <int D, int WM, int WN, int HG>
__global__ __launch_bounds__(64 * WM * WN) void sdpa_prefill_kernel(PrefillDev p) {
    constexpr int kThreads = 64 * WM * WN;
    constexpr int QB = WM / HG;           // 32-query blocks per workgroup
    constexpr int BLOCK_M = 32 * QB, BLOCK_N = 64 * WN;
    static_assert(WM % HG == 0, "waves split evenly over the heads of a workgroup");
    constexpr int KS = D / 16;            // contraction steps of Q K^T
    constexpr int DB = D / 32;            // 32-feature blocks of the output
    constexpr int KROW = D + 8;           // halfs per K row in LDS: 128-bit reads of 16 rows hit 64 distinct banks
    constexpr int VROW = D + 16;          // halfs per V row in LDS: the 4 rows of a transposing read sit 8 banks apart
    constexpr int NL = BLOCK_N * D / 8 / kThreads;  // 128-bit loads per thread per tile and tensor
    static_assert(WM * WN == 4 || WM * WN == 8, "four or eight waves per workgroup");
    static_assert(NL >= 1 && NL * 8 * kThreads == BLOCK_N * D, "tile loads must divide evenly");

    __shared__ __attribute__((aligned(16))) _Float16 lds_all[BLOCK_N * (KROW + VROW)];
    _Float16 *lds_k = lds_all;
    _Float16 *lds_v = lds_all + BLOCK_N * KROW;

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hb = lane >> 5, l32 = lane & 31;
    const int wm = w % WM, wn = w / WM;

    // workgroup -> (kv head fastest, so that consecutive workgroup ids, which the hardware deals
    // round-robin to the 8 XCDs, keep one kv head's K/V in one XCD's L2), longest query tiles first
    int id = blockIdx.x;
    const int kvh = id % p.Hkv;
    id /= p.Hkv;
    const int G = p.Hq / p.Hkv;
    const int gg = id % (G / HG);         // group of HG query heads of this kv head
    id /= (G / HG);
    const int qt = p.n_qtiles - 1 - (id % p.n_qtiles);
    const int b = id / p.n_qtiles;
    const int qh = kvh * G + gg * HG + (wm % HG);

    const int off = p.Sk - p.Sq;          // query i sees keys j <= i + off when causal
    const int q0 = qt * BLOCK_M + 32 * (wm / HG);  // first query of this wave
    const int my_q = q0 + l32;
    const _Float16 *qrow = p.q + (((int64_t)b * p.Hq + qh) * p.Sq + min(my_q, p.Sq - 1)) * D;
    const _Float16 *kbase = p.k + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    const _Float16 *vbase = p.v + (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;

    // Q^T fragments: query = lane % 32, features 16*ks + 8*hb .. +8
    half8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *reinterpret_cast<const half8_t *>(qrow + 16 * ks + 8 * hb);
    // Settle the Q loads here.  Otherwise the compiler must assume they may still be in flight at
    // the top of the tile loop and waits for vmcnt(0) at their first use there, which also waits
    // for the K/V prefetch issued a few instructions earlier and exposes its whole latency.
#pragma unroll
    for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[ks]));

    // key tiles this workgroup needs
    const int wg_q_last = min(qt * BLOCK_M + BLOCK_M, p.Sq) - 1;
    const int last_key = p.causal ? min(p.Sk - 1, wg_q_last + off) : p.Sk - 1;
    const int n_kt = last_key / BLOCK_N + 1;
    const int wave_q_last = min(q0 + 31, p.Sq - 1);

    float m_run = -INFINITY, l_run = 0.0f;
    float16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;

    u32x4 kpre[NL], vpre[NL];
    auto prefetch = [&](int kt) {
#pragma unroll
        for (int j = 0; j < NL; j++) {
            int c = j * kThreads + tid;
            int key = c / (D / 8), dc = c % (D / 8);
            int64_t row = min(kt * BLOCK_N + key, p.Sk - 1);
            kpre[j] = *reinterpret_cast<const u32x4 *>(kbase + row * p.kv_stride_t + dc * 8);
            vpre[j] = *reinterpret_cast<const u32x4 *>(vbase + row * p.kv_stride_t + dc * 8);
        }
    };
    prefetch(0);

    for (int kt = 0; kt < n_kt; kt++) {
        __syncthreads();  // everyone is done reading the previous tile
#pragma unroll
        for (int j = 0; j < NL; j++) {
            int c = j * kThreads + tid;
            int key = c / (D / 8), dc = c % (D / 8);
            *reinterpret_cast<u32x4 *>(&lds_k[key * KROW + dc * 8]) = kpre[j];
            *reinterpret_cast<u32x4 *>(&lds_v[key * VROW + dc * 8]) = vpre[j];
        }
        __syncthreads();
        if (kt + 1 < n_kt) prefetch(kt + 1);

        const int k_lo = kt * BLOCK_N + 64 * wn;  // first key of this wave's slice
        const bool active = k_lo < p.Sk && (!p.causal || k_lo <= wave_q_last + off);
        if (!active) continue;

        // ---- S^T = K Q^T : 2 key blocks of 32 x 32 queries -------------------------------------
        float16_t s[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s[kb][r] = 0.0f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                half8_t kf = *reinterpret_cast<const half8_t *>(&lds_k[(64 * wn + 32 * kb + l32) * KROW + 16 * ks + 8 * hb]);
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s[kb], 0, 0, 0);
            }
        }
        // ---- online softmax for query lane%32 over this lane's 32 keys ---------------------------
        const bool need_mask = (k_lo + 64 > p.Sk) || (p.causal && (k_lo + 63 > q0 + off));
        float tmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float x = s[kb][r] * p.scale_log2;
                if (need_mask) {
                    int key = k_lo + 32 * kb + 8 * (r >> 2) + 4 * hb + (r & 3);
                    bool vis = key < p.Sk && (!p.causal || key <= my_q + off);
                    x = vis ? x : -INFINITY;
                }
                s[kb][r] = x;
                tmax = fmaxf(tmax, x);
            }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // nothing visible yet: keep everything at zero
        const float alpha = fast_exp2(m_run - m_ref);
        float psum = 0.0f;
        half8_t pf[4];  // P^T fragments: contraction step st takes accumulator rows 8*(st%2)..+8 of block st/2
#pragma unroll
        for (int st = 0; st < 4; st++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float pv = fast_exp2(s[st >> 1][8 * (st & 1) + i] - m_ref);
                psum += pv;
                pf[st][i] = (_Float16)pv;
            }
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        // ---- O^T += V^T P^T ------------------------------------------------------------------------
        // This lane as a SOURCE of the transposing loads: key row (lane%16)/4 of a group of four,
        // features 16*(lane/16 % 2) + 4*(lane%4) of the 32-feature block.
        const _Float16 *vsrc = &lds_v[(64 * wn + 4 * hb + ((lane & 15) >> 2)) * VROW + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)];
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
    }

    // ---- merge the two lane halves' sums, then the WN key slices through LDS ---------------------
    l_run += __shfl_xor(l_run, 32, 64);
    if constexpr (WN > 1) {
        __syncthreads();  // the tiles are dead: reuse their space
        float *xo = reinterpret_cast<float *>(lds_all);  // [WN-1][WM][64 lanes][DB*16 + 2]
        constexpr int kPer = DB * 16 + 2;
        static_assert(sizeof(float) * (WN - 1) * WM * 64 * kPer <= sizeof(_Float16) * BLOCK_N * (KROW + VROW), "merge buffer");
        if (wn > 0) {
            float *mine = xo + (((size_t)(wn - 1) * WM + wm) * 64 + lane) * kPer;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) mine[db * 16 + r] = o[db][r];
            mine[DB * 16] = m_run;
            mine[DB * 16 + 1] = l_run;
        }
        __syncthreads();
        if (wn > 0) return;
#pragma unroll
        for (int other = 1; other < WN; other++) {
            const float *theirs = xo + (((size_t)(other - 1) * WM + wm) * 64 + lane) * kPer;
            const float m_o = theirs[DB * 16], l_o = theirs[DB * 16 + 1];
            const float mm = fmaxf(m_run, m_o);
            const float m_ref = (mm == -INFINITY) ? 0.0f : mm;
            const float fa = fast_exp2(m_run - m_ref), fb = fast_exp2(m_o - m_ref);
            l_run = l_run * fa + l_o * fb;
            m_run = mm;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] = o[db][r] * fa + theirs[db * 16 + r] * fb;
        }
    }
    if (my_q >= p.Sq) return;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    _Float16 *orow = p.out + (((int64_t)b * p.Hq + qh) * p.Sq + my_q) * D;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            half4_t h4;
#pragma unroll
            for (int i = 0; i < 4; i++) h4[i] = (_Float16)(o[db][4 * rq + i] * inv);
            *reinterpret_cast<half4_t *>(orow + 32 * db + 8 * rq + 4 * hb) = h4;
        }
}

template <int D, int WM, int WN, int HG>
int launch_cfg(const PrefillDev &p0, hipStream_t s) {
    PrefillDev p = p0;
    constexpr int BLOCK_M = 32 * WM / HG;
    if ((p.Hq / p.Hkv) % HG) return 2;
    p.n_qtiles = (p.Sq + BLOCK_M - 1) / BLOCK_M;
    int64_t wgs = (int64_t)p.B * (p.Hq / HG) * p.n_qtiles;
    if (wgs >= (1ll << 31)) return 2;
    hipLaunchKernelGGL((sdpa_prefill_kernel<D, WM, WN, HG>), dim3((unsigned)wgs), dim3(64 * WM * WN), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_prefill launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace

int launch_sdpa_prefill(const SdpaArgs &a, hipStream_t s) {
    if (a.q_dtype != TROCM_F16 || a.kv_fmt != TROCM_F16 || a.mask != nullptr) return 2;
    if (a.D != 128 && a.D != 64) return 2;
    if (a.Sq < 2 || a.Sk < 1 || a.Hq % a.Hkv) return 2;
    if (a.causal && a.Sk < a.Sq) return 2;  // some queries would see nothing: the generic kernel owns that case
    if (a.Sk >= (1ll << 30) || a.Sq >= (1ll << 30) || a.B >= (1ll << 20)) return 2;
    if ((a.kv_stride_b % 8) || (a.kv_stride_h % 8) || (a.kv_stride_t % 8)) return 2;  // 128-bit row loads
    if ((uintptr_t)a.q % 16 || (uintptr_t)a.k % 16 || (uintptr_t)a.v % 16 || (uintptr_t)a.out % 8) return 2;
    PrefillDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const _Float16 *)a.q;
    p.out = (_Float16 *)a.out;
    p.k = (const _Float16 *)a.k;
    p.v = (const _Float16 *)a.v;
    p.kv_stride_b = a.kv_stride_b, p.kv_stride_h = a.kv_stride_h, p.kv_stride_t = a.kv_stride_t;
    p.B = (int)a.B, p.Hq = (int)a.Hq, p.Hkv = (int)a.Hkv, p.Sq = (int)a.Sq, p.Sk = (int)a.Sk;
    p.causal = a.causal;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    // Shapes, named WM WN HG: 4 1 1 = four waves, 128 queries of one head; 2 2 1 = four waves, 64
    // queries, keys split two ways; 4 2 1 = eight waves, 128 queries, keys split two ways.
    // TROCM_PREFILL_SHAPE=<WM><WN><HG> forces one (experiments).
    static const int forced = getenv("TROCM_PREFILL_SHAPE") ? atoi(getenv("TROCM_PREFILL_SHAPE")) : 0;
    const int64_t G = a.Hq / a.Hkv;
    int shape = forced;
    if (!shape) {
        (void)G;
        int64_t wgs_421 = a.B * a.Hq * ((a.Sq + 127) / 128);
        shape = wgs_421 >= num_compute_units() ? 421 : 221;
    }
#define TROCM_PREFILL_CASES(DD)                                        \
    switch (shape) {                                                   \
        case 411: return launch_cfg<DD, 4, 1, 1>(p, s);                \
        case 221: return launch_cfg<DD, 2, 2, 1>(p, s);                \
        case 421: return launch_cfg<DD, 4, 2, 1>(p, s);                \
        default: return fail("unknown prefill shape %d", shape);       \
    }
    if (a.D == 128) {
        TROCM_PREFILL_CASES(128)
    }
    TROCM_PREFILL_CASES(64)
#undef TROCM_PREFILL_CASES
}

}  // namespace trocm
