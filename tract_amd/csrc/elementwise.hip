// The element-wise ops that sit beside the cache and attention in an exported decoder layer:
//   cast f32 <-> f16      (core `Cast`; cuda/src/kernels/array/cast.rs:21-47)
//   RotateHalf            (transformers/src/ops/apply_rope.rs:58-76)
//   ApplyRope             (transformers/src/ops/apply_rope.rs:169-176; strided / broadcast
//                          dispatch as cuda/src/kernels/nn/apply_rope.rs:59-129)
// All three are HBM-bound byte movers; results are bit-exact with the CPU ops:
//   y = x * cos + rotate_half(x) * sin, every operation rounded to the tensor's datum type
// (f16: product and sum are formed in f32 and rounded to f16 after each operation, which is how
// the CPU's f16 arithmetic works).  Compiled with -ffp-contract=off.
#include <hip/hip_fp16.h>
#include <string.h>
#include <type_traits>
#include "common.h"

namespace trocm {
namespace {

__device__ __forceinline__ float round_dt(float x, float *) { return x; }
// Round to f16 and back as its own instruction (see kv_quant.hip: a fused mixed-precision fma
// would lose the sign of a zero product).
__device__ __forceinline__ float round_dt(float x, __half *) {
    asm volatile("" : "+v"(x));
    return __half2float(__float2half_rn(x));
}
__device__ __forceinline__ float ld(const float *p) { return *p; }
__device__ __forceinline__ float ld(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ void st(float *p, float x) { *p = x; }
__device__ __forceinline__ void st(__half *p, float x) { *p = __float2half_rn(x); }  // x is already representable

struct Rope4 {
    int64_t shape[4];       // padded on the left with 1s
    int64_t in_s[4], cs_s[4], out_s[4];   // element strides; cs_s is 0 on broadcast axes
    int64_t half;
    int rotate_only;
};

// One thread per (row, i < half): both elements of the rotation pair.
template <typename T>
__global__ __launch_bounds__(256) void apply_rope_kernel(const T *__restrict__ x, const T *__restrict__ cs,
                                                          const T *__restrict__ sn, T *__restrict__ y, Rope4 p,
                                                          int64_t n_pairs) {
    int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n_pairs) return;
    const int64_t i = idx % p.half;
    int64_t r = idx / p.half;
    const int64_t i2 = r % p.shape[2];
    r /= p.shape[2];
    const int64_t i1 = r % p.shape[1];
    const int64_t i0 = r / p.shape[1];
    const int64_t xo = i0 * p.in_s[0] + i1 * p.in_s[1] + i2 * p.in_s[2];
    const int64_t yo = i0 * p.out_s[0] + i1 * p.out_s[1] + i2 * p.out_s[2];
    const float a = ld(x + xo + i * p.in_s[3]);
    const float b = ld(x + xo + (i + p.half) * p.in_s[3]);
    T *tag = nullptr;
    float lo, hi;
    if (p.rotate_only) {
        lo = -b;   // RotateHalf: [-x2, x1]
        hi = a;
    } else {
        const int64_t co = i0 * p.cs_s[0] + i1 * p.cs_s[1] + i2 * p.cs_s[2];
        const float c_lo = ld(cs + co + i * p.cs_s[3]), s_lo = ld(sn + co + i * p.cs_s[3]);
        const float c_hi = ld(cs + co + (i + p.half) * p.cs_s[3]), s_hi = ld(sn + co + (i + p.half) * p.cs_s[3]);
        lo = round_dt(__fadd_rn(round_dt(__fmul_rn(a, c_lo), tag), round_dt(__fmul_rn(-b, s_lo), tag)), tag);
        hi = round_dt(__fadd_rn(round_dt(__fmul_rn(b, c_hi), tag), round_dt(__fmul_rn(a, s_hi), tag)), tag);
    }
    st(y + yo + i * p.out_s[3], lo);
    st(y + yo + (i + p.half) * p.out_s[3], hi);
}

// Streaming accesses for data that is read or written once: non-temporal loads and stores keep it out
// of the caches' replacement order.
typedef uint32_t nt_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t nt_u32x2 __attribute__((ext_vector_type(2)));
template <int BYTES>
__device__ __forceinline__ void stream_copy_in(void *regs, const void *src) {
    if constexpr (BYTES == 16)
        *reinterpret_cast<nt_u32x4 *>(regs) = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4 *>(src));
    else
        *reinterpret_cast<nt_u32x2 *>(regs) = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x2 *>(src));
}
template <int BYTES>
__device__ __forceinline__ void stream_copy_out(void *dst, const void *regs) {
    if constexpr (BYTES == 16)
        __builtin_nontemporal_store(*reinterpret_cast<const nt_u32x4 *>(regs), reinterpret_cast<nt_u32x4 *>(dst));
    else
        __builtin_nontemporal_store(*reinterpret_cast<const nt_u32x2 *>(regs), reinterpret_cast<nt_u32x2 *>(dst));
}

// The same with 16-byte accesses: one thread per VW consecutive rotation pairs (VW = 8 halfs or 4
// floats).  Used when the innermost strides are 1 and everything is 16-byte aligned, which is every
// layout an exported decoder produces; the scalar kernel above moved 1.4 TB/s on a prefill chunk.
template <typename T>
__global__ __launch_bounds__(256) void apply_rope_vec_kernel(const T *__restrict__ x, const T *__restrict__ cs,
                                                              const T *__restrict__ sn, T *__restrict__ y, Rope4 p,
                                                              int64_t n_groups) {
    constexpr int VW = 16 / sizeof(T);
    int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n_groups) return;
    const int64_t gph = p.half / VW;       // groups per half row
    const int64_t i = (idx % gph) * VW;
    int64_t r = idx / gph;
    const int64_t i2 = r % p.shape[2];
    r /= p.shape[2];
    const int64_t i1 = r % p.shape[1];
    const int64_t i0 = r / p.shape[1];
    const T *xr = x + i0 * p.in_s[0] + i1 * p.in_s[1] + i2 * p.in_s[2];
    T *yr = y + i0 * p.out_s[0] + i1 * p.out_s[1] + i2 * p.out_s[2];
    T a[VW], b[VW], c_lo[VW], s_lo[VW], c_hi[VW], s_hi[VW], lo[VW], hi[VW];
    stream_copy_in<16>(a, xr + i);
    stream_copy_in<16>(b, xr + i + p.half);
    if (!p.rotate_only) {
        const int64_t co = i0 * p.cs_s[0] + i1 * p.cs_s[1] + i2 * p.cs_s[2];
        *reinterpret_cast<uint4 *>(c_lo) = *reinterpret_cast<const uint4 *>(cs + co + i);
        *reinterpret_cast<uint4 *>(s_lo) = *reinterpret_cast<const uint4 *>(sn + co + i);
        *reinterpret_cast<uint4 *>(c_hi) = *reinterpret_cast<const uint4 *>(cs + co + i + p.half);
        *reinterpret_cast<uint4 *>(s_hi) = *reinterpret_cast<const uint4 *>(sn + co + i + p.half);
    }
    T *tag = nullptr;
#pragma unroll
    for (int j = 0; j < VW; j++) {
        const float fa = ld(&a[j]), fb = ld(&b[j]);
        float l, h;
        if (p.rotate_only) {
            l = -fb, h = fa;
        } else {
            l = round_dt(__fadd_rn(round_dt(__fmul_rn(fa, ld(&c_lo[j])), tag), round_dt(__fmul_rn(-fb, ld(&s_lo[j])), tag)), tag);
            h = round_dt(__fadd_rn(round_dt(__fmul_rn(fb, ld(&c_hi[j])), tag), round_dt(__fmul_rn(fa, ld(&s_hi[j])), tag)), tag);
        }
        st(&lo[j], l);
        st(&hi[j], h);
    }
    stream_copy_out<16>(yr + i, lo);
    stream_copy_out<16>(yr + i + p.half, hi);
}

template <typename S, typename Dd>
__global__ __launch_bounds__(256) void cast_kernel(const S *__restrict__ src, Dd *__restrict__ dst, size_t n) {
    for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += (size_t)gridDim.x * 1024)
    if (i + 4 <= n && ((uintptr_t)src % (4 * sizeof(S)) == 0) && ((uintptr_t)dst % (4 * sizeof(Dd)) == 0)) {
        S in[4];
        Dd out[4];
        stream_copy_in<4 * sizeof(S)>(in, src + i);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float f = ld(&in[j]);
            st(&out[j], f);   // f32 -> f16 rounds to nearest even; f16 -> f32 is exact
        }
        stream_copy_out<4 * sizeof(Dd)>(dst + i, out);
    } else {
        for (size_t j = i; j < n && j < i + 4; j++) st(dst + j, ld(src + j));
    }
}

}  // namespace

int launch_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n, hipStream_t s) {
    if (n == 0) return 0;
    if (src_dtype == dst_dtype) {
        TROCM_HIP(hipMemcpyAsync(dst, src, n * elem_bytes(src_dtype), hipMemcpyDeviceToDevice, s));
        return 0;
    }
    size_t blocks = (n + 1023) / 1024;
    // at most 64 workgroups per compute unit, whose threads then take several trips (64 Mi elements f32 -> f16: one trip
    // per thread 69.3 us, 128 per compute unit 65.0, 64: 64.2, 32: 64.1, 16: 65.0)
    if (blocks > (size_t)num_compute_units() * 64) blocks = (size_t)num_compute_units() * 64;
    TROCM_REQUIRE(blocks < (1ull << 31), "cast: tensor too large");
    if (src_dtype == TROCM_F32)
        hipLaunchKernelGGL((cast_kernel<float, __half>), dim3((unsigned)blocks), dim3(256), 0, s, (const float *)src, (__half *)dst, n);
    else
        hipLaunchKernelGGL((cast_kernel<__half, float>), dim3((unsigned)blocks), dim3(256), 0, s, (const __half *)src, (float *)dst, n);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("cast launch failed: %s", hipGetErrorString(e));
    return 0;
}

int launch_apply_rope(const void *x, const void *cos, const void *sin, void *y, int dtype, int rank,
                      const int64_t *shape, const int64_t *in_strides, const int64_t *cs_strides,
                      const int64_t *out_strides, int rotate_only, hipStream_t s) {
    Rope4 p;
    memset(&p, 0, sizeof(p));
    const int pad = 4 - rank;
    int64_t n = 1;
    for (int d = 0; d < 4; d++) {
        p.shape[d] = d < pad ? 1 : shape[d - pad];
        n *= p.shape[d];
    }
    int64_t dense = 1;
    for (int d = 3; d >= 0; d--) {
        const int64_t dflt = dense;
        dense *= p.shape[d];
        if (d < pad) continue;
        p.in_s[d] = in_strides ? in_strides[d - pad] : dflt;
        p.out_s[d] = out_strides ? out_strides[d - pad] : dflt;
        p.cs_s[d] = cs_strides ? cs_strides[d - pad] : dflt;
    }
    p.half = p.shape[3] / 2;
    p.rotate_only = rotate_only;
    if (n == 0) return 0;
    const int64_t n_pairs = n / 2;
    const int64_t vw = dtype == TROCM_F32 ? 4 : 8, eb = dtype == TROCM_F32 ? 4 : 2;
    bool vec = p.in_s[3] == 1 && p.out_s[3] == 1 && (rotate_only || p.cs_s[3] == 1) && p.half % vw == 0 &&
               (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 && (rotate_only || ((uintptr_t)cos % 16 == 0 && (uintptr_t)sin % 16 == 0));
    for (int d = 0; d < 3 && vec; d++)
        vec = (p.in_s[d] * eb) % 16 == 0 && (p.out_s[d] * eb) % 16 == 0 && (rotate_only || (p.cs_s[d] * eb) % 16 == 0);
    if (vec) {
        const int64_t n_groups = n_pairs / vw;
        const int64_t vblocks = (n_groups + 255) / 256;
        TROCM_REQUIRE(vblocks < (1ll << 31), "apply_rope: tensor too large");
        if (dtype == TROCM_F32)
            hipLaunchKernelGGL((apply_rope_vec_kernel<float>), dim3((unsigned)vblocks), dim3(256), 0, s, (const float *)x,
                               (const float *)cos, (const float *)sin, (float *)y, p, n_groups);
        else
            hipLaunchKernelGGL((apply_rope_vec_kernel<__half>), dim3((unsigned)vblocks), dim3(256), 0, s, (const __half *)x,
                               (const __half *)cos, (const __half *)sin, (__half *)y, p, n_groups);
        hipError_t ev = hipGetLastError();
        if (ev != hipSuccess) return fail("apply_rope launch failed: %s", hipGetErrorString(ev));
        return 0;
    }
    const int64_t blocks = (n_pairs + 255) / 256;
    TROCM_REQUIRE(blocks < (1ll << 31), "apply_rope: tensor too large");
    if (dtype == TROCM_F32)
        hipLaunchKernelGGL((apply_rope_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s, (const float *)x,
                           (const float *)cos, (const float *)sin, (float *)y, p, n_pairs);
    else
        hipLaunchKernelGGL((apply_rope_kernel<__half>), dim3((unsigned)blocks), dim3(256), 0, s, (const __half *)x,
                           (const __half *)cos, (const __half *)sin, (__half *)y, p, n_pairs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("apply_rope launch failed: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace trocm
