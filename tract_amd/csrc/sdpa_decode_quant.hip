// Split-K flash-decode over a block-quantised KV cache (Q8_0 / Q4_0, head_dim 128), with
// the dequantisation fused into the loads.  Same decomposition as the f16 kernel
// (sdpa_decode.hip): grid (splits, kv_heads, batch), 4 waves per workgroup, 32-token tiles,
// K codes staged through LDS for the transposed read, V codes straight from HBM.
//
// Codes become f16 without a per-element conversion instruction: one v_perm_b32 puts two
// code bytes under the exponent byte 0x64, i.e. forms the halves (1024 + u), u = code + 128 for Q8_0
// (the cache's code plane holds exactly that byte) and u = nibble for Q4_0.
//   QK : dot2 accumulates sum q_i (1024 + u_i) per 32-element block; the constant part
//        (1152 or 1032 times the block sum of q, computed once per workgroup) is subtracted
//        and the block scale d applied:  s += d * (dot - bias * qsum).
//   PV : (1024 + u) - bias is exact in f16 and (code * d) rounded to f16 is the reference's
//        dequantised value; two tokens share a dot2 against the f16 pair (p_a, p_b).
// The reference dequantises to f16 ((code * d) rounded to f16, q4_0.rs:82-95) before its f32
// attention; V is formed exactly so, for K the product with d stays in f32 (a difference below
// half an f16 ulp per element).
//
// Roofline: HBM-bound on paper (34/32 or 18/32 bytes per element) but the vector ALU work
// per byte is 2-4x that of f16, so these kernels are ALU-limited before they are
// bandwidth-limited; algorithmic bytes per launch = 2*B*Hkv*T*D*(34|18)/32 + Q + O.
#include "decode_common.h"

namespace trocm {
namespace {

constexpr int kD = 128;
constexpr int kNB = kD / 32;  // blocks per row

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}
// halves (0x6400 | byte0, 0x6400 | byte1) and (0x6400 | byte2, 0x6400 | byte3) of x
__device__ __forceinline__ half2_t magic_lo(uint32_t x) { return as_half2(perm(0x64646464u, x, 0x04010400u)); }
__device__ __forceinline__ half2_t magic_hi(uint32_t x) { return as_half2(perm(0x64646464u, x, 0x04030402u)); }

template <int FMT>
struct QTraits;
template <>
struct QTraits<TROCM_Q8_0> {
    static constexpr int kRowBytes = kD;      // code bytes per token row
    static constexpr float kBias = 1152.0f;   // 1024 + 128
    typedef uint2 vcode_t;                    // 8 codes per lane in the PV phase
};
template <>
struct QTraits<TROCM_Q4_0> {
    static constexpr int kRowBytes = kD / 2;
    static constexpr float kBias = 1032.0f;   // 1024 + 8
    typedef uint32_t vcode_t;                 // 4 bytes = 8 nibbles per lane
};

template <int CPR>
__device__ __forceinline__ int qrot(int row) {
    return CPR == 8 ? (row >> 1) : (row >> 2);
}

// Streaming (non-temporal) loads of the code planes: K and V are read once per launch, and keeping them
// out of the caches' replacement order is worth 8-9 % of a decode launch.
template <typename V>
__device__ __forceinline__ V stream_load(const char *ptr);
template <>
__device__ __forceinline__ uint32_t stream_load<uint32_t>(const char *ptr) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(ptr));
}
template <>
__device__ __forceinline__ uint2 stream_load<uint2>(const char *ptr) {
    const uint64_t raw = __builtin_nontemporal_load(reinterpret_cast<const uint64_t *>(ptr));
    uint2 v;
    v.x = (uint32_t)raw, v.y = (uint32_t)(raw >> 32);
    return v;
}

template <int FMT, int G>
__global__ __launch_bounds__(kThreads, G <= 4 ? 2 : 1) void sdpa_decode_q_kernel(DecodeDev p) {
    typedef QTraits<FMT> Q;
    typedef typename Q::vcode_t vcode_t;
    constexpr int D = kD;
    constexpr int RB = Q::kRowBytes;       // 128 / 64
    constexpr int CPR = RB / 16;           // 8 / 4
    constexpr int HC = CPR / 2;            // code chunks per half row: 4 / 2
    constexpr int KL = kTile * CPR / 64;   // 4 / 2
    constexpr int QC = D * 2 / 16;         // 16-byte chunks of one f16 query row: 16
    constexpr int EPL = 8;
    constexpr int VI = kTile / 4;
    constexpr int SB = kNB * 2;            // scale bytes per token row

    __shared__ u32x4 lds_k[kWaves][kTile * CPR];
    __shared__ u32x4 lds_q[G * QC];
    __shared__ float lds_qsum[G * kNB];    // bias * sum of q over each block
    __shared__ float lds_p[kWaves][kTile * G];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, and the compiler is told so
    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;

    {
        const u32x4 *qg = reinterpret_cast<const u32x4 *>(p.q + ((int64_t)b * p.Hq + (int64_t)kvh * p.g_real) * (D * 2));
        for (int i = tid; i < G * QC; i += kThreads) lds_q[i] = qg[min(i / QC, p.g_real - 1) * QC + i % QC];
        if (tid < G * kNB) {
            const __half *qh = reinterpret_cast<const __half *>(p.q) + ((int64_t)b * p.Hq + (int64_t)kvh * p.g_real) * D +
                               min(tid / kNB, p.g_real - 1) * D + (tid % kNB) * 32;
            float sum = 0.0f;
            for (int i = 0; i < 32; i++) sum += __half2float(qh[i]);
            lds_qsum[tid] = sum * Q::kBias;
        }
    }
    __syncthreads();

    const int64_t bh_off = (int64_t)b * p.kv_stride_b + (int64_t)kvh * p.kv_stride_h;
    const int64_t sc_off = (int64_t)b * p.sc_stride_b + (int64_t)kvh * p.sc_stride_h;
    const char *kbase = p.k + bh_off, *vbase = p.v + bh_off;
    const char *ksbase = p.k_scales + sc_off, *vsbase = p.v_scales + sc_off;
    const int n_tiles = (p.T + kTile - 1) / kTile;
    const int tile_begin = split * p.tiles_per_split;
    const int tile_end = min(n_tiles, tile_begin + p.tiles_per_split);
    const int last_tok = p.T - 1;

    float m[G], l[G], o[G][EPL];
#pragma unroll
    for (int h = 0; h < G; h++) {
        m[h] = -INFINITY;
        l[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; e++) o[h][e] = 0.0f;
    }

    const int rg = lane >> 4, j16 = lane & 15;
    const int qk_row = lane >> 1, qk_half = lane & 1;
    const int vblk = j16 >> 2;  // block of this lane's V columns
    uint32_t k_off[KL], k_slot[KL];
#pragma unroll
    for (int j = 0; j < KL; j++) {
        int L = j * 64 + lane;
        int row = L / CPR, c = L % CPR;
        k_off[j] = (uint32_t)row * RB + (uint32_t)c * 16u;
        k_slot[j] = row * CPR + ((c + qrot<CPR>(row)) & (CPR - 1));
    }

    u32x4 kreg[KL];
    uint32_t ksreg;  // the two block scales of this lane's half row
    vcode_t vreg[VI];
    uint16_t vsreg[VI];
    auto issue_k = [&](int tile) {
        const int t0 = tile * kTile;
        const char *base = kbase + (int64_t)t0 * RB;
        if (t0 + kTile <= p.T) {
#pragma unroll
            for (int j = 0; j < KL; j++) kreg[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + k_off[j]));
            ksreg = *reinterpret_cast<const uint32_t *>(ksbase + (int64_t)(t0 + qk_row) * SB + qk_half * 4);
        } else {
#pragma unroll
            for (int j = 0; j < KL; j++) {
                int L = j * 64 + lane;
                int row = min(L / CPR, last_tok - t0), c = L % CPR;
                kreg[j] = *reinterpret_cast<const u32x4 *>(base + (uint32_t)row * RB + (uint32_t)c * 16u);
            }
            ksreg = *reinterpret_cast<const uint32_t *>(ksbase + (int64_t)min(t0 + qk_row, last_tok) * SB + qk_half * 4);
        }
    };
    auto issue_v = [&](int tile) {
        const int t0 = tile * kTile;
#pragma unroll
        for (int i = 0; i < VI; i++) {
            int tok = min(t0 + 4 * i + rg, last_tok);
            vreg[i] = stream_load<vcode_t>(vbase + (int64_t)tok * RB + j16 * (int)sizeof(vcode_t));
            vsreg[i] = *reinterpret_cast<const uint16_t *>(vsbase + (int64_t)tok * SB + vblk * 2);
        }
    };

    int tile = tile_begin + w;
    if (tile < tile_end) {
        issue_k(tile);
        issue_v(tile);
    }
    const u32x4 *lds_krow = &lds_k[w][qk_row * CPR];
    const int qk_rot = qrot<CPR>(qk_row) + qk_half * HC;

    for (; tile < tile_end; tile += kWaves) {
        const int t0 = tile * kTile;
#pragma unroll
        for (int j = 0; j < KL; j++) lds_k[w][k_slot[j]] = kreg[j];
        const uint32_t ks = ksreg;
        const bool more = tile + kWaves < tile_end;
        if (more) issue_k(tile + kWaves);

        // ---- scores: this lane covers blocks [qk_half*2, qk_half*2 + 2) of token t0+qk_row
        float s[G];
#pragma unroll
        for (int h = 0; h < G; h++) s[h] = 0.0f;
#pragma unroll
        for (int bl = 0; bl < kNB / 2; bl++) {
            const int blk = qk_half * (kNB / 2) + bl;  // block index within the row
            float acc[G];
#pragma unroll
            for (int h = 0; h < G; h++) acc[h] = 0.0f;
            if constexpr (FMT == TROCM_Q8_0) {
                // block = 2 code chunks of 16 codes; chunk cc pairs with q chunks 2cc, 2cc+1 of the block
#pragma unroll
                for (int cc = 0; cc < 2; cc++) {
                    u32x4 kc = lds_krow[(bl * 2 + cc + qk_rot) & (CPR - 1)];
                    uint32_t kw[4] = {kc.x, kc.y, kc.z, kc.w};   // the plane holds code + 128
#pragma unroll
                    for (int h = 0; h < G; h++) {
                        u32x4 q0 = lds_q[h * QC + blk * 4 + cc * 2], q1 = lds_q[h * QC + blk * 4 + cc * 2 + 1];
                        uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
                        for (int wd = 0; wd < 4; wd++) {
                            acc[h] = __builtin_amdgcn_fdot2(magic_lo(kw[wd]), as_half2(qw[2 * wd]), acc[h], false);
                            acc[h] = __builtin_amdgcn_fdot2(magic_hi(kw[wd]), as_half2(qw[2 * wd + 1]), acc[h], false);
                        }
                        __builtin_amdgcn_sched_barrier(0);  // keep the next head's LDS reads from piling up in registers
                    }
                }
            } else {
                // block = 1 chunk of 16 bytes: low nibbles are elements 0..15, high nibbles 16..31
                u32x4 kc = lds_krow[(bl + qk_rot) & (CPR - 1)];
                uint32_t kx[4] = {kc.x, kc.y, kc.z, kc.w};
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int wd = 0; wd < 4; wd++) {
                    lo[wd] = kx[wd] & 0x0F0F0F0Fu;
                    hi[wd] = (kx[wd] >> 4) & 0x0F0F0F0Fu;
                }
#pragma unroll
                for (int h = 0; h < G; h++) {
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        u32x4 q0 = lds_q[h * QC + blk * 4 + half * 2], q1 = lds_q[h * QC + blk * 4 + half * 2 + 1];
                        uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
                        for (int wd = 0; wd < 4; wd++) {
                            uint32_t c4 = half ? hi[wd] : lo[wd];
                            acc[h] = __builtin_amdgcn_fdot2(magic_lo(c4), as_half2(qw[2 * wd]), acc[h], false);
                            acc[h] = __builtin_amdgcn_fdot2(magic_hi(c4), as_half2(qw[2 * wd + 1]), acc[h], false);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            float d = __half2float(__ushort_as_half((uint16_t)(bl ? (ks >> 16) : (ks & 0xffffu))));
#pragma unroll
            for (int h = 0; h < G; h++) s[h] = fmaf(d, acc[h] - lds_qsum[h * kNB + blk], s[h]);
        }
        const bool valid = (t0 + qk_row) < p.T;
        float pr[G], alpha[G];
        bool moved = false;
#pragma unroll
        for (int h = 0; h < G; h++) {
            float full = s[h] + dpp_f<kSwapPairs>(s[h]);
            float sv = valid ? full * p.scale_log2 : -INFINITY;
            float m_new = fmaxf(m[h], wave_max(sv));
            alpha[h] = fast_exp2(m[h] - m_new);
            pr[h] = fast_exp2(sv - m_new);
            l[h] = l[h] * alpha[h] + pr[h];
            moved = moved || (m_new != m[h]);
            m[h] = m_new;
        }
        if (moved) {  // wave-uniform: the running maxima rarely move after the first tiles
#pragma unroll
            for (int h = 0; h < G; h++)
#pragma unroll
                for (int e = 0; e < EPL; e++) o[h][e] *= alpha[h];
        }
        if (qk_half == 0) {
#pragma unroll
            for (int h = 0; h < G; h++) lds_p[w][qk_row * G + h] = pr[h];
        }
        // ---- O += P V with fused dequantisation, two tokens per dot2 ---------------------------
        // Tokens 4*(2j)+rg and 4*(2j+1)+rg of this lane are paired: their code bytes are interleaved
        // (one v_perm per two elements) and turned into halves 1024+u; a packed subtract (exact) and
        // a packed multiply form (code_a * d_a, code_b * d_b) rounded once to f16 -- the reference's
        // dequantised values (q4_0.rs:82-95).  dot2 with the f16 pair (p_a, p_b) accumulates in f32.
#pragma unroll
        for (int j = 0; j < VI / 2; j++) {
            const int ia = 2 * j, ib = 2 * j + 1;
            const half2_t dpair = as_half2((uint32_t)vsreg[ia] | ((uint32_t)vsreg[ib] << 16));
            const half2_t bias = {(_Float16)Q::kBias, (_Float16)Q::kBias};
            half2_t pp[G];
#pragma unroll
            for (int h = 0; h < G; h++) {
                pp[h][0] = (_Float16)lds_p[w][(4 * ia + rg) * G + h];
                pp[h][1] = (_Float16)lds_p[w][(4 * ib + rg) * G + h];
            }
            uint32_t wa[2], wb[2];
            if constexpr (FMT == TROCM_Q8_0) {
                wa[0] = vreg[ia].x, wa[1] = vreg[ia].y;   // the plane holds code + 128
                wb[0] = vreg[ib].x, wb[1] = vreg[ib].y;
            } else {
                wa[0] = vreg[ia] & 0x0F0F0F0Fu, wa[1] = (vreg[ia] >> 4) & 0x0F0F0F0Fu;
                wb[0] = vreg[ib] & 0x0F0F0F0Fu, wb[1] = (vreg[ib] >> 4) & 0x0F0F0F0Fu;
            }
#pragma unroll
            for (int wd = 0; wd < 2; wd++) {
                // bytes (a0, b0, a1, b1) and (a2, b2, a3, b3) of this word's four elements
                const uint32_t t01 = perm(wa[wd], wb[wd], 0x01050004u), t23 = perm(wa[wd], wb[wd], 0x03070206u);
                half2_t v2[4] = {magic_lo(t01), magic_hi(t01), magic_lo(t23), magic_hi(t23)};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const half2_t vd = (v2[i] - bias) * dpair;
#pragma unroll
                    for (int h = 0; h < G; h++) o[h][4 * wd + i] = __builtin_amdgcn_fdot2(vd, pp[h], o[h][4 * wd + i], false);
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one token pair at a time: keeps the register count down
        }
        if (more) issue_v(tile + kWaves);
    }

    // ---- merge row groups, waves, splits: same scheme as the f16 kernel -----------------------
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
    __shared__ float comb[kWaves][G * D + 2 * G];
    if (rg == 0) {
#pragma unroll
        for (int h = 0; h < G; h++)
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                // output column of accumulator e: Q8_0 lanes own 8 consecutive columns; Q4_0 lanes own
                // 4 low-nibble columns and the 4 columns 16 further on of their block
                int col = FMT == TROCM_Q8_0 ? j16 * 8 + e : vblk * 32 + (j16 & 3) * 4 + (e & 3) + 16 * (e >> 2);
                comb[w][h * D + col] = o[h][e];
            }
    }
    if (lane == 0) {
#pragma unroll
        for (int h = 0; h < G; h++) {
            comb[w][G * D + h] = m[h];
            comb[w][G * D + G + h] = l[h];
        }
    }
    __syncthreads();

    const int64_t bh = (int64_t)b * p.Hkv + kvh;
    __half *out = reinterpret_cast<__half *>(p.out) + ((int64_t)b * p.Hq + (int64_t)kvh * p.g_real) * D;
    for (int idx = tid; idx < G * D; idx += kThreads) {
        int h = idx / D;
        float mm = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) mm = fmaxf(mm, comb[ww][G * D + h]);
        float acc = 0.0f, ll = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
            float f = fast_exp2(comb[ww][G * D + h] - mm);
            acc += comb[ww][idx] * f;
            ll += comb[ww][G * D + G + h] * f;
        }
        if (p.nsplit == 1) {
            if (h < p.g_real) out[idx] = __float2half_rn(ll > 0.0f ? acc / ll : 0.0f);
        } else if (p.counters == nullptr) {
            int64_t slot = bh * p.nsplit + split;
            p.part_o[slot * (G * D) + idx] = acc;
            if ((idx % D) == 0) {
                p.part_ml[slot * (2 * G) + h] = mm;
                p.part_ml[slot * (2 * G) + G + h] = ll;
            }
        } else {   // write-through stores: visible device-wide when they complete (see tail_merge)
            int64_t slot = bh * p.nsplit + split;
            __hip_atomic_store(&p.part_o[slot * (G * D) + idx], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((idx % D) == 0) {
                __hip_atomic_store(&p.part_ml[slot * (2 * G) + h], mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&p.part_ml[slot * (2 * G) + G + h], ll, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (p.nsplit == 1 || p.counters == nullptr) return;
    tail_merge<__half, D, G>(p, p.counters + bh, p.nsplit, bh * p.nsplit, 1, out, tid);
}

template <int FMT, int G>
int launch_one(const DecodeDev &p, dim3 grid, hipStream_t s) {
    hipLaunchKernelGGL((sdpa_decode_q_kernel<FMT, G>), grid, dim3(kThreads), 0, s, p);
    if (p.nsplit > 1 && p.counters == nullptr)
        hipLaunchKernelGGL((sdpa_decode_merge_kernel<__half, kD, G>), dim3(grid.y, grid.z, p.g_real), dim3(kD), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_decode (quantised KV) launch failed: %s", hipGetErrorString(e));
    return 0;
}

template <int FMT>
int launch_fmt(const DecodeDev &p, int G, dim3 grid, hipStream_t s) {
    switch (G) {
        case 1: return launch_one<FMT, 1>(p, grid, s);
        case 2: return launch_one<FMT, 2>(p, grid, s);
        case 4: return launch_one<FMT, 4>(p, grid, s);
        case 8: return launch_one<FMT, 8>(p, grid, s);
    }
    return 2;
}

}  // namespace

int launch_sdpa_decode_quant(const SdpaArgs &a, hipStream_t s) {
    if (a.Sq != 1 || a.mask != nullptr) return 2;
    if (a.kv_fmt != TROCM_Q8_0 && a.kv_fmt != TROCM_Q4_0) return 2;
    if (a.q_dtype != TROCM_F16 || a.D != kD) return 2;
    if (a.Hq % a.Hkv) return 2;
    const int64_t g_real = a.Hq / a.Hkv;
    const bool mfma = decode_mfma_group(g_real) != 0;   // grouped heads: the MFMA formulation (sdpa_decode_mfma.hip)
    if (g_real > 8 && !mfma) return 2;
    // a fused append (the step's new token, f16 rows [B, Hkv, 1, D] like q): only the block-scaling MFMA bodies take it
    if (a.k_new && (!mfma || !decode_quant_appends_in_kernel(g_real, a.scale) || a.v_new == nullptr || a.new_pos >= 0 ||
                    (uintptr_t)a.k_new % 16 || (uintptr_t)a.v_new % 16))
        return 2;
    // q and the new key rotated on the way in: the (head, block) bodies of the MFMA formulation only
    if (a.rope_cos && (!a.rope_sin || !a.k_new || !mfma || !decode_quant_rotates_in_kernel(g_real) || (uintptr_t)a.rope_cos % 16 ||
                       (uintptr_t)a.rope_sin % 16 || (a.rope_stride_b * 2) % 16))
        return 2;
    const int64_t G = g_real <= 2 ? g_real : g_real <= 4 ? 4 : 8;   // the instantiation that runs it
    if (a.kv_stride_t != a.D) return 2;  // cache planes: token rows are dense
    if ((uintptr_t)a.k % 16 || (uintptr_t)a.v % 16 || (uintptr_t)a.q % 16 || (uintptr_t)a.k_scales % 4 ||
        (uintptr_t)a.v_scales % 4)
        return 2;
    if (a.Sk <= 0 || a.Sk > (1ll << 30) || a.B > 65535 || a.Hkv > 65535) return 2;
    int64_t BH = a.B * a.Hkv;
    const int64_t rb = a.kv_fmt == TROCM_Q8_0 ? kD : kD / 2;
    // plane strides: the logical element strides scale with the bytes per token row
    int64_t cap_h = a.kv_stride_h / a.D, cap_b = a.kv_stride_b / a.D;  // in token rows
    if ((cap_h * rb) % 16 || (cap_b * rb) % 16) return 2;

    if (mfma) {
        DecodeDev p;
        memset(&p, 0, sizeof(p));
        p.q = (const char *)a.q, p.out = (char *)a.out, p.k = (const char *)a.k, p.v = (const char *)a.v;
        p.kv_stride_b = cap_b * rb, p.kv_stride_h = cap_h * rb, p.kv_stride_t = rb;
        p.k_scales = (const char *)a.k_scales, p.v_scales = (const char *)a.v_scales;
        p.sc_stride_b = cap_b * kNB * 2, p.sc_stride_h = cap_h * kNB * 2;
        p.T = (int)a.Sk;
        p.Hq = (int)a.Hq, p.Hkv = (int)a.Hkv, p.g_real = (int)g_real;
        p.scale_log2 = a.scale * 1.4426950408889634f;
        p.k_new = (const char *)a.k_new, p.v_new = (const char *)a.v_new;
        p.new_pos = a.k_new ? (int)a.Sk - 1 : -1;
        if (a.rope_cos) p.rope_cos = (const char *)a.rope_cos, p.rope_sin = (const char *)a.rope_sin, p.rope_stride_b = a.rope_stride_b * 2;
        return launch_sdpa_decode_quant_mfma(p, a.kv_fmt, a.B, a.workspace, a.workspace_bytes, s);
    }
    if (a.rope_cos) return 2;
    int n_tiles = (int)((a.Sk + kTile - 1) / kTile);
    int nsplit = fit_decode_splits(choose_decode_splits(BH, G, n_tiles, 2), BH, G, a.D, a.workspace, a.workspace_bytes);
    int tps = (n_tiles + nsplit - 1) / nsplit;
    nsplit = (n_tiles + tps - 1) / tps;
    DecodeDev p;
    memset(&p, 0, sizeof(p));
    p.q = (const char *)a.q;
    p.out = (char *)a.out;
    p.k = (const char *)a.k;
    p.v = (const char *)a.v;
    p.kv_stride_b = cap_b * rb;
    p.kv_stride_h = cap_h * rb;
    p.kv_stride_t = rb;
    p.k_scales = (const char *)a.k_scales;
    p.v_scales = (const char *)a.v_scales;
    p.sc_stride_b = cap_b * kNB * 2;
    p.sc_stride_h = cap_h * kNB * 2;
    p.T = (int)a.Sk;
    p.tiles_per_split = tps;
    p.nsplit = nsplit;
    p.Hq = (int)a.Hq;
    p.Hkv = (int)a.Hkv;
    p.g_real = (int)g_real;
    p.scale_log2 = a.scale * 1.4426950408889634f;
    p.part_ml = (float *)((char *)a.workspace + kWsCounterBytes);
    p.part_o = p.part_ml + (size_t)BH * nsplit * 2 * G;
    // few splits: the last workgroup of a (batch, kv head) to arrive merges them, no second launch
    static const int tail = getenv("TROCM_DECODE_TAIL_MERGE") ? atoi(getenv("TROCM_DECODE_TAIL_MERGE")) : 1;
    if (tail && nsplit > 1 && nsplit <= kTailMergeMax && BH <= (int64_t)(kWsCounterBytes / sizeof(int))) p.counters = (int *)a.workspace;
    dim3 grid(nsplit, (unsigned)a.Hkv, (unsigned)a.B);
    return a.kv_fmt == TROCM_Q8_0 ? launch_fmt<TROCM_Q8_0>(p, (int)G, grid, s) : launch_fmt<TROCM_Q4_0>(p, (int)G, grid, s);
}

}  // namespace trocm
