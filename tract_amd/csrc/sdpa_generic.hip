// Shape-generic scaled-dot-product attention for gfx950: any head_dim <= 512, any
// q_len / kv_len / group size, f32 or f16, optional additive mask or causal masking,
// strided K/V.  It is the catch-all behind the specialised decode and prefill kernels
// (the role Sdpa's exploded einsum+softmax graph plays on tract's CPU,
// transformers/src/ops/sdpa.rs:131-227) and is written for exactness, not speed: natural
// exponent, two passes (row maximum first), f32 accumulation.
//
// One wavefront per query row.  Pass 1: lane-per-key scores and the row maximum.  Pass 2,
// per 64-key tile: p = exp(s - max) goes through LDS, then lane d accumulates output
// columns d, d+64, ...
#include <hip/hip_fp16.h>
#include "common.h"

namespace trocm {
namespace {

struct GenericDev {
    const void *q, *k, *v, *mask;
    const void *k_scales, *v_scales;  // quantised K/V: f16 scale planes
    int kv_fmt;
    void *out;
    int64_t B, Hq, Hkv, Sq, Sk, D;
    int64_t kv_stride_b, kv_stride_h, kv_stride_t;  // elements
    int64_t mask_b, mask_h;
    float scale;
    int causal;
};

__device__ __forceinline__ float ld(const float *p) { return *p; }
__device__ __forceinline__ float ld(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ void st(float *p, float x) { *p = x; }
__device__ __forceinline__ void st(__half *p, float x) { *p = __float2half_rn(x); }

// Element (token j, column d) of a K or V plane of one (batch, kv head).  Plain formats: a row
// of T; quantised formats: code and block scale, dequantised as code * d in f32
// (linalg/src/frame/block_quant/q4_0.rs:82-95, q8_1.rs:50-63).
template <typename T>
struct KvReader {
    const T *rows;
    const uint8_t *codes;
    const uint16_t *scales;
    int64_t stride_t;  // elements between token rows (plain) -- quantised rows are dense
    int fmt, D;
    __device__ __forceinline__ float at(int64_t j, int d) const {
        if (fmt == TROCM_Q8_0) {
            float sc = __half2float(__ushort_as_half(scales[j * (D / 32) + d / 32]));
            return (float)((int)codes[j * D + d] - 128) * sc;   // the plane holds code + 128
        }
        if (fmt == TROCM_Q4_0) {
            float sc = __half2float(__ushort_as_half(scales[j * (D / 32) + d / 32]));
            int e = d & 31;
            uint8_t byte = codes[j * (D / 2) + (d / 32) * 16 + (e & 15)];
            int nib = e < 16 ? (byte & 15) : (byte >> 4);
            return (float)(nib - 8) * sc;
        }
        return ld(rows + j * stride_t + d);
    }
};

template <typename T>
__device__ __forceinline__ KvReader<T> make_reader(const GenericDev &p, const void *plane, const void *scales, int64_t b,
                                                   int64_t kvh) {
    KvReader<T> r;
    r.fmt = p.kv_fmt, r.D = (int)p.D, r.stride_t = p.kv_stride_t;
    r.rows = nullptr, r.codes = nullptr, r.scales = nullptr;
    if (p.kv_fmt == TROCM_Q8_0 || p.kv_fmt == TROCM_Q4_0) {
        int64_t row0 = (b * p.kv_stride_b + kvh * p.kv_stride_h) / p.D;  // first token row of this (batch, head)
        int64_t rb = p.kv_fmt == TROCM_Q8_0 ? p.D : p.D / 2;
        r.codes = (const uint8_t *)plane + row0 * rb;
        r.scales = (const uint16_t *)scales + row0 * (p.D / 32);
    } else {
        r.rows = (const T *)plane + b * p.kv_stride_b + kvh * p.kv_stride_h;
    }
    return r;
}

template <typename T>
__global__ __launch_bounds__(64) void sdpa_generic_kernel(GenericDev p) {
    __shared__ float lds_q[512];
    __shared__ float lds_p[64];
    const int lane = threadIdx.x;
    int64_t row = blockIdx.x;
    const int64_t i = row % p.Sq;
    row /= p.Sq;
    const int64_t qh = row % p.Hq;
    const int64_t b = row / p.Hq;
    const int64_t G = p.Hq / p.Hkv;
    const int64_t kvh = qh / G;
    const int D = (int)p.D;

    const T *q = (const T *)p.q + ((b * p.Hq + qh) * p.Sq + i) * p.D;
    const KvReader<T> k = make_reader<T>(p, p.k, p.k_scales, b, kvh);
    const KvReader<T> v = make_reader<T>(p, p.v, p.v_scales, b, kvh);
    T *out = (T *)p.out + ((b * p.Hq + qh) * p.Sq + i) * p.D;
    const T *mask = nullptr;
    if (p.mask) {
        int64_t mb = b < p.mask_b - 1 ? b : p.mask_b - 1;
        int64_t mh = qh < p.mask_h - 1 ? qh : p.mask_h - 1;
        mask = (const T *)p.mask + ((mb * p.mask_h + mh) * p.Sq + i) * p.Sk;
    }
    for (int d = lane; d < D; d += 64) lds_q[d] = ld(q + d);
    __syncthreads();

    // keys visible to query i: j <= i + (Sk - Sq) when causal
    int64_t n_vis = p.Sk;
    if (p.causal) {
        int64_t lim = i + (p.Sk - p.Sq) + 1;
        n_vis = lim < 0 ? 0 : (lim < p.Sk ? lim : p.Sk);
    }
    auto score = [&](int64_t j) {
        float acc = 0.0f;
        for (int d = 0; d < D; d++) acc = fmaf(lds_q[d], k.at(j, d), acc);
        acc *= p.scale;
        if (mask) acc += ld(mask + j);
        return acc;
    };
    float mx = -INFINITY;
    for (int64_t j = lane; j < n_vis; j += 64) mx = fmaxf(mx, score(j));
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) mx = fmaxf(mx, __shfl_xor(mx, s, 64));

    float o[8];
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = 0.0f;
    float l = 0.0f;
    if (mx > -INFINITY) {
        for (int64_t j0 = 0; j0 < n_vis; j0 += 64) {
            int64_t j = j0 + lane;
            float pj = j < n_vis ? expf(score(j) - mx) : 0.0f;
            l += pj;
            __syncthreads();
            lds_p[lane] = pj;
            __syncthreads();
            int64_t n = n_vis - j0 < 64 ? n_vis - j0 : 64;
            for (int64_t jj = 0; jj < n; jj++) {
                float pp = lds_p[jj];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    int d = lane + 64 * e;
                    if (d < D) o[e] = fmaf(pp, v.at(j0 + jj, d), o[e]);
                }
            }
        }
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) l += __shfl_xor(l, s, 64);
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
        int d = lane + 64 * e;
        if (d < D) st(out + d, l > 0.0f ? o[e] / l : 0.0f);
    }
}

}  // namespace

int launch_sdpa_generic(const SdpaArgs &a, hipStream_t s) {
    const bool quant = a.kv_fmt == TROCM_Q8_0 || a.kv_fmt == TROCM_Q4_0;
    TROCM_REQUIRE(quant || a.q_dtype == a.kv_fmt, "generic sdpa: Q and K/V must share a dtype");
    TROCM_REQUIRE(!quant || (a.D % 32 == 0 && a.kv_stride_t == a.D), "generic sdpa: quantised K/V needs dense rows and head_dim %% 32 == 0");
    TROCM_REQUIRE(a.D >= 1 && a.D <= 512, "generic sdpa: head_dim %lld not in 1..512", (long long)a.D);
    int64_t rows = a.B * a.Hq * a.Sq;
    if (rows == 0) return 0;
    TROCM_REQUIRE(rows < (1ll << 31), "generic sdpa: too many query rows");
    GenericDev p;
    p.q = a.q, p.k = a.k, p.v = a.v, p.mask = a.mask, p.out = a.out;
    p.k_scales = a.k_scales, p.v_scales = a.v_scales, p.kv_fmt = a.kv_fmt;
    p.B = a.B, p.Hq = a.Hq, p.Hkv = a.Hkv, p.Sq = a.Sq, p.Sk = a.Sk, p.D = a.D;
    p.kv_stride_b = a.kv_stride_b, p.kv_stride_h = a.kv_stride_h, p.kv_stride_t = a.kv_stride_t;
    p.mask_b = a.mask_b, p.mask_h = a.mask_h;
    p.scale = a.scale;
    p.causal = a.causal;
    if (a.q_dtype == TROCM_F16)
        hipLaunchKernelGGL(sdpa_generic_kernel<__half>, dim3((unsigned)rows), dim3(64), 0, s, p);
    else
        hipLaunchKernelGGL(sdpa_generic_kernel<float>, dim3((unsigned)rows), dim3(64), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_generic launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace trocm
