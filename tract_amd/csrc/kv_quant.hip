// Q8_0 / Q4_0 block quantisation on KV append, canonical export and dequantisation.
//
// Stored bytes must equal what tract's CPU block quantisers produce
// (linalg/src/frame/block_quant/q4_0.rs:19-45, q8_1.rs:20-48 without the `sum`
// field), so every floating-point step is spelled out: no contraction of a*b+c (this
// file is compiled with -ffp-contract=off and uses the _rn intrinsics), IEEE division,
// round-half-away for Q8 codes, truncation for Q4 codes, RNE for the f16 scale.
//
// Device layout (private): a code plane with one row per token ([D] bytes for Q8_0, each code + 128 -- offset binary:
// the attention kernels put a code byte under an exponent byte to make the f16 integer 1024 + byte, and with the sign
// bit already flipped they do not have to flip it for every byte they read;
// [D/2] bytes = 16 canonical nibble bytes per block for Q4_0) and a scale plane with
// D/32 f16 per token, so that decode can read both with aligned 128-bit loads.
//
// Each block is scanned by one thread in element order: the quantiser's "first element
// with strictly largest |v|" rule is order dependent, and a 32-element block is 64-128
// bytes, so one lane reads whole 128-bit words.  The work is HBM-bound (reads 2-4 bytes
// and writes ~1 byte per element).
#include <hip/hip_fp16.h>
#include <stdlib.h>
#include "common.h"
#include "quant_block.h"

namespace trocm {
namespace {

// (A signalling NaN is quieted on the way in: v_max3_f32 / v_min3_f32 answer NaN for one, and the next instruction of
// the chain, ignoring that NaN, would have lost the two values that shared an instruction with it.  Quiet or
// signalling, a NaN is skipped by the scan and codes as 0, so nothing else changes.)
__device__ __forceinline__ float load_elem(const float *p) { return __builtin_canonicalizef(*p); }
__device__ __forceinline__ float load_elem(const __half *p) { return __half2float(*p); }

__device__ __forceinline__ void store_out(float *p, float x) { *p = x; }
__device__ __forceinline__ void store_out(__half *p, float x) { *p = __ushort_as_half(f32_to_f16_bits(x)); }

template <typename SrcT>
__device__ __forceinline__ void load_block(const SrcT *p, int64_t stride, bool vec, float (&v)[32]) {
    if (vec) {  // dense and 16-byte aligned: whole 128-bit words
        constexpr int kPerWord = 16 / sizeof(SrcT);
        const uint4 *w = reinterpret_cast<const uint4 *>(p);
#pragma unroll
        for (int i = 0; i < 32 / kPerWord; i++) {
            uint4 x = w[i];
            const SrcT *e = reinterpret_cast<const SrcT *>(&x);
#pragma unroll
            for (int j = 0; j < kPerWord; j++) v[i * kPerWord + j] = load_elem(e + j);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) v[i] = load_elem(p + i * stride);
    }
}

struct QuantAppendDev {
    int fmt;
    int vec;
    int64_t B, H, S, D;
    int64_t ss[4];
    int64_t cap, t0;
    const void *src;
    uint8_t *codes;
    uint16_t *scales;
    int64_t n_blocks;
    int nb_shift;   // log2(D / 32) when that is a power of two, else -1
};

__device__ __forceinline__ void quant_store_block(const QuantAppendDev &a, const float (&v)[32], int64_t row, int64_t nb, int64_t blk) {
    if (a.fmt == TROCM_Q8_0) {
        uint32_t c[8];
        uint16_t d = quant_q8(v, c);
        uint4 *dst = reinterpret_cast<uint4 *>(a.codes + row * a.D + blk * 32);
        constexpr uint32_t x = 0x80808080u;   // the plane holds code + 128
        dst[0] = make_uint4(c[0] ^ x, c[1] ^ x, c[2] ^ x, c[3] ^ x);
        dst[1] = make_uint4(c[4] ^ x, c[5] ^ x, c[6] ^ x, c[7] ^ x);
        a.scales[row * nb + blk] = d;
    } else {
        uint32_t c[4];
        uint16_t d = quant_q4(v, c);
        *reinterpret_cast<uint4 *>(a.codes + row * (a.D / 2) + blk * 16) = make_uint4(c[0], c[1], c[2], c[3]);
        a.scales[row * nb + blk] = d;
    }
}

template <typename SrcT>
__device__ __forceinline__ void quant_one_block(const QuantAppendDev &a, const SrcT *p, int64_t row, int64_t nb, int64_t blk) {
    float v[32];
    load_block(p, a.ss[3], a.vec != 0, v);
    quant_store_block(a, v, row, nb, blk);
}

// Grid (chunks of a (batch, head) row's blocks, batch * heads), one block per thread: the position of a block inside
// its row is one 32-bit division (a shift when head_dim / 32 is a power of two); with a flat index over all blocks the
// three 64-bit divisions were 45 % of the kernel's instructions.  Dense sources have a loop of their own: with the
// choice between 128-bit and element loads inside one loop the same launch measured 82 us instead of 75 us.
template <typename SrcT>
__device__ __forceinline__ void quant_append_body(const QuantAppendDev &a) {
    const uint32_t nb = (uint32_t)(a.D / 32);
    const uint32_t per_row = (uint32_t)a.S * nb;
    const uint32_t first = blockIdx.x * blockDim.x + threadIdx.x, step = gridDim.x * blockDim.x;
    constexpr int kWords = 32 * sizeof(SrcT) / 16;
    for (int64_t bh = blockIdx.y; bh < a.B * a.H; bh += gridDim.y) {
        const int64_t b = bh / a.H, h = bh % a.H;   // (scalar: once per workgroup trip)
        const SrcT *src_row = (const SrcT *)a.src + b * a.ss[0] + h * a.ss[1];
        const int64_t row0 = bh * a.cap + a.t0;
        if (a.vec) {
            if (first >= per_row) continue;
            for (uint32_t i = first; i < per_row; i += step) {
                const uint32_t t = a.nb_shift >= 0 ? i >> a.nb_shift : i / nb;
                const uint32_t blk = i - t * nb;
                const uint4 *p = reinterpret_cast<const uint4 *>(src_row + (int64_t)t * a.ss[2] + (int64_t)blk * 32);
                uint4 w[kWords];
#pragma unroll
                for (int k = 0; k < kWords; k++) w[k] = p[k];
                float v[32];
                constexpr int kPerWord = 16 / sizeof(SrcT);
#pragma unroll
                for (int k = 0; k < kWords; k++) {
                    const SrcT *e = reinterpret_cast<const SrcT *>(&w[k]);
#pragma unroll
                    for (int q = 0; q < kPerWord; q++) v[k * kPerWord + q] = load_elem(e + q);
                }
                quant_store_block(a, v, row0 + t, nb, blk);
            }
            continue;
        }
        for (uint32_t i = first; i < per_row; i += step) {
            const uint32_t t = a.nb_shift >= 0 ? i >> a.nb_shift : i / nb;
            const uint32_t blk = i - t * nb;
            quant_one_block(a, src_row + (int64_t)t * a.ss[2] + (int64_t)blk * 32 * a.ss[3], row0 + t, nb, blk);
        }
    }
}

template <typename SrcT>
__global__ __launch_bounds__(256) void quant_append_kernel(QuantAppendDev a) {
    quant_append_body<SrcT>(a);
}
// K and V of the same shape in one launch: blockIdx.z selects the tensor.
template <typename SrcT>
__global__ __launch_bounds__(256) void quant_append_pair_kernel(QuantAppendDev k, QuantAppendDev v) {
    if (blockIdx.z == 0) quant_append_body<SrcT>(k);
    else quant_append_body<SrcT>(v);
}

// One token per sequence into per-sequence planes: grid (sequences, 2 = K / V).
template <typename SrcT>
__global__ __launch_bounds__(256) void quant_append_ragged_kernel(int fmt, const QuantAppendSeq *__restrict__ table,
                                                                  const SrcT *__restrict__ k_new, const SrcT *__restrict__ v_new,
                                                                  int64_t H, int64_t D, int vec) {
    const QuantAppendSeq e = table[blockIdx.x];
    const bool is_v = blockIdx.y != 0;
    const SrcT *src = (is_v ? v_new : k_new) + (int64_t)blockIdx.x * H * D;
    uint8_t *codes = (uint8_t *)(is_v ? e.v_codes : e.k_codes);
    uint16_t *scales = (uint16_t *)(is_v ? e.v_scales : e.k_scales);
    const int64_t nb = D / 32;
    for (int64_t idx = threadIdx.x; idx < H * nb; idx += blockDim.x) {
        const int64_t blk = idx % nb, h = idx / nb;
        float v[32];
        load_block(src + h * D + blk * 32, 1, vec != 0, v);
        const int64_t row = h * e.cap + e.t0;
        if (fmt == TROCM_Q8_0) {
            uint32_t c[8];
            const uint16_t d = quant_q8(v, c);
            uint4 *dst = reinterpret_cast<uint4 *>(codes + row * D + blk * 32);
            constexpr uint32_t x = 0x80808080u;   // the plane holds code + 128
            dst[0] = make_uint4(c[0] ^ x, c[1] ^ x, c[2] ^ x, c[3] ^ x);
            dst[1] = make_uint4(c[4] ^ x, c[5] ^ x, c[6] ^ x, c[7] ^ x);
            scales[row * nb + blk] = d;
        } else {
            uint32_t c[4];
            const uint16_t d = quant_q4(v, c);
            *reinterpret_cast<uint4 *>(codes + row * (D / 2) + blk * 16) = make_uint4(c[0], c[1], c[2], c[3]);
            scales[row * nb + blk] = d;
        }
    }
}

// Canonical export: [B,H,len, nb * (2 + code bytes)], 2-byte aligned stores.
__global__ __launch_bounds__(256) void quant_export_kernel(int fmt, int64_t BH, int64_t len, int64_t cap, int64_t D,
                                                           const uint8_t *__restrict__ codes,
                                                           const uint16_t *__restrict__ scales,
                                                           uint16_t *__restrict__ dst) {
    int64_t nb = D / 32;
    int64_t total = BH * len * nb;
    int cw = fmt == TROCM_Q8_0 ? 16 : 8;  // code bytes / 2
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t blk = idx % nb;
        int64_t rem = idx / nb;
        int64_t t = rem % len;
        int64_t bh = rem / len;
        int64_t row = bh * cap + t;
        const uint16_t *c = reinterpret_cast<const uint16_t *>(codes + (row * nb + blk) * (cw * 2));
        uint16_t *o = dst + ((bh * len + t) * nb + blk) * (1 + cw);
        o[0] = scales[row * nb + blk];
        const uint16_t flip = fmt == TROCM_Q8_0 ? 0x8080 : 0;   // Q8_0 planes hold code + 128
        for (int i = 0; i < cw; i++) o[1 + i] = c[i] ^ flip;
    }
}

// Canonical import, the inverse of the export: blocks [B,H,n, nb * (2 + code bytes)] are split into
// the code and scale planes at tokens [t0, t0 + n) of every (batch, head) row.
__global__ __launch_bounds__(256) void quant_import_kernel(int fmt, int64_t BH, int64_t n, int64_t pitch, int64_t t0,
                                                           int64_t D, const uint16_t *__restrict__ src,
                                                           uint8_t *__restrict__ codes, uint16_t *__restrict__ scales) {
    int64_t nb = D / 32;
    int64_t total = BH * n * nb;
    int cw = fmt == TROCM_Q8_0 ? 16 : 8;  // code bytes / 2
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t blk = idx % nb;
        int64_t rem = idx / nb;
        int64_t t = rem % n;
        int64_t bh = rem / n;
        int64_t row = bh * pitch + t0 + t;
        const uint16_t *i16 = src + ((bh * n + t) * nb + blk) * (1 + cw);
        uint16_t *c = reinterpret_cast<uint16_t *>(codes + (row * nb + blk) * (cw * 2));
        scales[row * nb + blk] = i16[0];
        const uint16_t flip = fmt == TROCM_Q8_0 ? 0x8080 : 0;   // Q8_0 planes hold code + 128
        for (int i = 0; i < cw; i++) c[i] = i16[1 + i] ^ flip;
    }
}

// Canonical blocks from a dense tensor (BlockQuant::quant_f32/quant_f16 as a tensor op).
template <typename SrcT>
__global__ __launch_bounds__(256) void block_quant_kernel(int fmt, const SrcT *__restrict__ src, int64_t n_blocks,
                                                          bool vec, uint16_t *__restrict__ dst) {
    int cw = fmt == TROCM_Q8_0 ? 16 : 8;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n_blocks;
         idx += (int64_t)gridDim.x * blockDim.x) {
        float v[32];
        load_block(src + idx * 32, 1, vec, v);
        uint16_t *o = dst + idx * (1 + cw);
        if (fmt == TROCM_Q8_0) {
            uint32_t c[8];
            o[0] = quant_q8(v, c);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                o[1 + 2 * i] = (uint16_t)(c[i] & 0xffff);
                o[2 + 2 * i] = (uint16_t)(c[i] >> 16);
            }
        } else {
            uint32_t c[4];
            o[0] = quant_q4(v, c);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                o[1 + 2 * i] = (uint16_t)(c[i] & 0xffff);
                o[2 + 2 * i] = (uint16_t)(c[i] >> 16);
            }
        }
    }
}

// BlockQuant::dequant_f32 / dequant_f16 (block_quant/mod.rs:78-108; q4_0.rs:82-95, q8_1.rs:50-63):
// the product is formed in the output type: for f16 the f32 product is rounded to f16.
template <typename DstT>
__global__ __launch_bounds__(256) void block_dequant_kernel(int fmt, const uint8_t *__restrict__ blocks,
                                                            int64_t n_blocks, DstT *__restrict__ dst) {
    int bb = fmt == TROCM_Q8_0 ? 34 : 18;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n_blocks;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const uint8_t *q = blocks + idx * bb;
        float d = __half2float(__ushort_as_half((uint16_t)(q[0] | (q[1] << 8))));
        DstT *o = dst + idx * 32;
        if (fmt == TROCM_Q8_0) {
            for (int i = 0; i < 32; i++) store_out(o + i, __fmul_rn((float)(int8_t)q[2 + i], d));
        } else {
            for (int j = 0; j < 16; j++) {
                int lo = q[2 + j] & 0xf, hi = q[2 + j] >> 4;
                store_out(o + j, __fmul_rn((float)(lo - 8), d));
                store_out(o + j + 16, __fmul_rn((float)(hi - 8), d));
            }
        }
    }
}

// BlockQuant::simulate_precision_loss (block_quant/mod.rs:130-154): every block of 32 goes through the quantiser and
// straight back through the dequantiser of the tensor's own type; no block bytes are written.  In place when dst == src
// (a thread has read its whole block before it stores).
template <typename T>
__global__ __launch_bounds__(256) void block_simulate_kernel(int fmt, const T *__restrict__ src, int64_t n_blocks, bool vec,
                                                             T *__restrict__ dst) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n_blocks;
         idx += (int64_t)gridDim.x * blockDim.x) {
        float v[32];
        load_block(src + idx * 32, 1, vec, v);
        T *o = dst + idx * 32;
        if (fmt == TROCM_Q8_0) {
            uint32_t c[8];
            const float d = __half2float(__ushort_as_half(quant_q8(v, c)));
#pragma unroll
            for (int i = 0; i < 32; i++) store_out(o + i, __fmul_rn((float)(int8_t)((c[i >> 2] >> (8 * (i & 3))) & 0xff), d));
        } else {
            uint32_t c[4];
            const float d = __half2float(__ushort_as_half(quant_q4(v, c)));
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int byte = (c[j >> 2] >> (8 * (j & 3))) & 0xff;
                store_out(o + j, __fmul_rn((float)((byte & 0xf) - 8), d));
                store_out(o + j + 16, __fmul_rn((float)((byte >> 4) - 8), d));
            }
        }
    }
}

int grid_for(int64_t n) {
    int64_t blocks = (n + 255) / 256;
    int64_t cap = (int64_t)num_compute_units() * 16;
    return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("%s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

}  // namespace

// The device-side description of one append, and the grid (gx, gy) that covers it.
static int describe_quant_append(const QuantAppend &a, QuantAppendDev &d, int64_t &gx, int64_t &gy) {
    TROCM_REQUIRE(a.D % 32 == 0, "quantised KV cache needs head_dim %% 32 == 0, got %lld", (long long)a.D);
    d.fmt = a.fmt;
    d.B = a.B, d.H = a.H, d.S = a.S, d.D = a.D;
    for (int i = 0; i < 4; i++) d.ss[i] = a.ss[i];
    d.cap = a.cap, d.t0 = a.t0;
    d.src = a.src;
    d.codes = (uint8_t *)a.codes;
    d.scales = (uint16_t *)a.scales;
    d.n_blocks = a.B * a.H * a.S * (a.D / 32);
    size_t es = elem_bytes(a.src_dtype);
    // 128-bit loads need a dense innermost axis and every block start on a 16-byte boundary
    // (blocks are 32 elements = 64 or 128 bytes, so only the base and outer strides matter).
    bool vec = a.ss[3] == 1 && ((uintptr_t)a.src % 16 == 0);
    for (int i = 0; i < 3 && vec; i++) vec = (a.ss[i] * (int64_t)es) % 16 == 0;
    d.vec = vec;
    TROCM_REQUIRE(a.S * (a.D / 32) < (1ll << 31), "quant_append: %lld tokens of %lld blocks per (batch, head) row exceed the 32-bit index",
                  (long long)a.S, (long long)(a.D / 32));
    const int64_t nb = a.D / 32;
    d.nb_shift = -1;
    for (int sh = 0; sh < 16; sh++)
        if (nb == (1ll << sh)) d.nb_shift = sh;
    const int64_t per_row = a.S * nb, bh = a.B * a.H;
    // One block per thread whatever the size.  A fixed number of workgroups whose threads walk over several blocks was
    // measured against it on a 16384-token prefill (8 x 8 heads): 16 workgroups per compute unit and 4 blocks per thread
    // 82.6 us (Q8_0) / 66.6 us (Q4_0), with the next block requested before the current one is worked on 81.8 / 67.1
    // (two blocks ahead 86 / 72: fewer waves fit), a contiguous run of blocks per workgroup 87.5 / 70.3, one block per
    // thread 75-76 / 62-63.  The loops in the kernel only serve launches beyond the grid limits.
    gx = std::min<int64_t>((per_row + 255) / 256, 1 << 22);
    gy = bh < 65535 ? bh : 65535;
    return 0;
}

int launch_quant_append(const QuantAppend &a, hipStream_t s) {
    QuantAppendDev d;
    int64_t gx, gy;
    if (describe_quant_append(a, d, gx, gy)) return 1;
    if (d.n_blocks == 0) return 0;
    if (a.src_dtype == TROCM_F16)
        hipLaunchKernelGGL(quant_append_kernel<__half>, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, d);
    else
        hipLaunchKernelGGL(quant_append_kernel<float>, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, d);
    return check_launch("quant_append");
}

int launch_quant_append_pair(const QuantAppend &k, const QuantAppend &v, hipStream_t s) {
    if (k.src_dtype != v.src_dtype || k.B != v.B || k.H != v.H || k.S != v.S || k.D != v.D) return 2;
    QuantAppendDev dk, dv;
    int64_t gx, gy, gx2, gy2;
    if (describe_quant_append(k, dk, gx, gy) || describe_quant_append(v, dv, gx2, gy2)) return 1;
    if (dk.n_blocks == 0) return 0;
    if (k.src_dtype == TROCM_F16)
        hipLaunchKernelGGL(quant_append_pair_kernel<__half>, dim3((unsigned)gx, (unsigned)gy, 2), dim3(256), 0, s, dk, dv);
    else
        hipLaunchKernelGGL(quant_append_pair_kernel<float>, dim3((unsigned)gx, (unsigned)gy, 2), dim3(256), 0, s, dk, dv);
    return check_launch("quant_append_pair");
}

int launch_quant_append_ragged(int fmt, int src_dtype, int64_t n_seq, int64_t H, int64_t D, const QuantAppendSeq *table,
                               const void *k_new, const void *v_new, hipStream_t s) {
    if (n_seq == 0) return 0;
    const int vec = (uintptr_t)k_new % 16 == 0 && (uintptr_t)v_new % 16 == 0;   // rows of D elements, D % 32 == 0
    const int threads = H * (D / 32) >= 256 ? 256 : 64;
    if (src_dtype == TROCM_F16)
        hipLaunchKernelGGL(quant_append_ragged_kernel<__half>, dim3((unsigned)n_seq, 2), dim3(threads), 0, s, fmt, table,
                           (const __half *)k_new, (const __half *)v_new, H, D, vec);
    else
        hipLaunchKernelGGL(quant_append_ragged_kernel<float>, dim3((unsigned)n_seq, 2), dim3(threads), 0, s, fmt, table,
                           (const float *)k_new, (const float *)v_new, H, D, vec);
    return check_launch("quant_append_ragged");
}

int launch_quant_export(int fmt, int64_t B, int64_t H, int64_t len, int64_t cap, int64_t D, const void *codes,
                        const void *scales, void *dst, hipStream_t s) {
    int64_t total = B * H * len * (D / 32);
    if (total == 0) return 0;
    hipLaunchKernelGGL(quant_export_kernel, dim3(grid_for(total)), dim3(256), 0, s, fmt, B * H, len, cap, D,
                       (const uint8_t *)codes, (const uint16_t *)scales, (uint16_t *)dst);
    return check_launch("quant_export");
}

int launch_quant_import(int fmt, int64_t B, int64_t H, int64_t n, int64_t pitch, int64_t t0, int64_t D, const void *blocks,
                        void *codes, void *scales, hipStream_t s) {
    int64_t total = B * H * n * (D / 32);
    if (total == 0) return 0;
    hipLaunchKernelGGL(quant_import_kernel, dim3(grid_for(total)), dim3(256), 0, s, fmt, B * H, n, pitch, t0, D,
                       (const uint16_t *)blocks, (uint8_t *)codes, (uint16_t *)scales);
    return check_launch("quant_import");
}

int launch_block_quant(int fmt, const void *src, int src_dtype, size_t n_elems, void *dst, hipStream_t s) {
    int64_t nb = (int64_t)(n_elems / 32);
    if (nb == 0) return 0;
    bool vec = (uintptr_t)src % 16 == 0;
    if (src_dtype == TROCM_F16)
        hipLaunchKernelGGL(block_quant_kernel<__half>, dim3(grid_for(nb)), dim3(256), 0, s, fmt, (const __half *)src,
                           nb, vec, (uint16_t *)dst);
    else
        hipLaunchKernelGGL(block_quant_kernel<float>, dim3(grid_for(nb)), dim3(256), 0, s, fmt, (const float *)src, nb,
                           vec, (uint16_t *)dst);
    return check_launch("block_quant");
}

int launch_block_simulate(int fmt, const void *src, void *dst, int dtype, size_t n_elems, hipStream_t s) {
    int64_t nb = (int64_t)(n_elems / 32);
    if (nb == 0) return 0;
    bool vec = (uintptr_t)src % 16 == 0;
    if (dtype == TROCM_F16)
        hipLaunchKernelGGL(block_simulate_kernel<__half>, dim3(grid_for(nb)), dim3(256), 0, s, fmt, (const __half *)src, nb, vec,
                           (__half *)dst);
    else
        hipLaunchKernelGGL(block_simulate_kernel<float>, dim3(grid_for(nb)), dim3(256), 0, s, fmt, (const float *)src, nb, vec,
                           (float *)dst);
    return check_launch("block_simulate");
}

int launch_block_dequant(int fmt, const void *blocks, size_t n_elems, void *dst, int dst_dtype, hipStream_t s) {
    int64_t nb = (int64_t)(n_elems / 32);
    if (nb == 0) return 0;
    if (dst_dtype == TROCM_F16)
        hipLaunchKernelGGL(block_dequant_kernel<__half>, dim3(grid_for(nb)), dim3(256), 0, s, fmt,
                           (const uint8_t *)blocks, nb, (__half *)dst);
    else
        hipLaunchKernelGGL(block_dequant_kernel<float>, dim3(grid_for(nb)), dim3(256), 0, s, fmt,
                           (const uint8_t *)blocks, nb, (float *)dst);
    return check_launch("block_dequant");
}

}  // namespace trocm
