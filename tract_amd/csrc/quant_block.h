// The Q8_0 / Q4_0 block quantisers as device functions (linalg/src/frame/block_quant/q4_0.rs:19-45, q8_1.rs:20-48
// without the `sum` field), shared by the append kernels and by the decode kernels that quantise a step's new token
// themselves.  The stored bytes must equal the CPU quantisers', so no a*b+c may be contracted into an fma, whatever
// the file is compiled with: every product that an addition follows passes through an empty asm, which no contraction
// can cross (a pragma in these functions would not do: the _rn helpers are inline functions of the HIP headers, and
// their bodies keep the translation unit's setting).
#pragma once
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace trocm {
namespace {

// f32 -> f16, round to nearest even, as its own instruction.  The empty asm keeps the
// compiler from folding a preceding multiply into a mixed-precision fma whose +0 addend
// would turn a -0 product into +0 (the reference keeps the sign of zero).
__device__ __forceinline__ uint16_t f32_to_f16_bits(float x) {
    asm volatile("" : "+v"(x));
    return __half_as_ushort(__float2half_rn(x));
}
// a * b rounded to f32, and kept apart from whatever is added to it
__device__ __forceinline__ float product(float a, float b) {
    float p = __fmul_rn(a, b);
    asm("" : "+v"(p));
    return p;
}
// Rust `f32 as i8`: truncate toward zero, saturate, NaN -> 0.  v_cvt_i32_f32 does the first and the last itself
// (it truncates, saturates at the 32-bit range and turns NaN into 0); what is left is the clamp to 8 bits.
__device__ __forceinline__ int cvt_i32_rz_sat(float x) {
    int r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(x));   // (a C cast may assume the value is in range)
    return r;
}
__device__ __forceinline__ int sat_i8(float x) { return max(-128, min(127, cvt_i32_rz_sat(x))); }   // (one v_med3_i32)

// f32::round() followed by the saturating cast: half away from zero, as the conversion (which truncates) of
// x + copysign(0.49999997, x) with the addition rounded to nearest even.  0.49999997 is the float below 0.5: for a
// fraction below one half the sum stays under the next integer, at exactly one half the sum lies midway between two
// floats and ties to the even one, which is the integer; from 2^23 on x + 0.49999997 rounds back to x.  The sum truncates
// to round(x) for every float (all 2^23 mantissas of every exponent from 2^-3 to 2^24 were compared on the host; below
// 2^-3 the sum stays under 1, above 2^25 it is x; inf saturates and NaN gives 0 either way).
__device__ __forceinline__ int round_half_away_sat_i8(float x) {
    return sat_i8(__fadd_rn(x, __builtin_copysignf(0.49999997f, x)));
}

// Signed value of the first element with strictly largest magnitude (q4_0.rs:27-34): the element order decides.
__device__ __forceinline__ float signed_first_absmax_in_order(const float (&v)[32]) {
    float amax = 0.0f, mx = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float a = fabsf(v[i]);
        if (amax < a) {
            amax = a;
            mx = v[i];
        }
    }
    return mx;
}

// The same value without the ordered scan where the order cannot matter: the largest and the smallest element (NaN
// ignored, as the scan's comparison ignores it) are one v_max3 / v_min3 per two elements; whichever has the larger
// magnitude is the answer.  Equal magnitudes (a +x and a -x, all zeros, nothing but NaN) go through the scan.
__device__ __forceinline__ float signed_first_absmax(const float (&v)[32]) {
    float hi = v[0], lo = v[0];
#pragma unroll
    for (int i = 1; i < 32; i++) {
        hi = fmaxf(hi, v[i]);
        lo = fminf(lo, v[i]);
    }
    if (hi > -lo) return hi;
    if (-lo > hi) return lo;
    return signed_first_absmax_in_order(v);
}

// Q8: returns the f16 scale bits, codes packed 4 per word in element order.
__device__ __forceinline__ uint16_t quant_q8(const float (&v)[32], uint32_t (&codes)[8]) {
    float mx = signed_first_absmax(v);
    float scale = __fdiv_rn(mx, 127.0f);                               // q8_1.rs:39
    float r = (scale == 0.0f) ? 0.0f : __fdiv_rn(1.0f, scale);         // q8_1.rs:40
#pragma unroll
    for (int w = 0; w < 8; w++) {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            int c = round_half_away_sat_i8(product(v[w * 4 + b], r));  // q8_1.rs:45
            word |= (uint32_t)(c & 0xff) << (8 * b);
        }
        codes[w] = word;
    }
    return f32_to_f16_bits(scale);
}

// Q4: byte j = code(elem j) | code(elem j+16) << 4 (q4_0.rs:39-44, helpers.rs:62-68).
__device__ __forceinline__ uint16_t quant_q4(const float (&v)[32], uint32_t (&codes)[4]) {
    float mx = signed_first_absmax(v);
    float scale = __fdiv_rn(mx, -8.0f);                                // q4_0.rs:35
    float r = (scale == 0.0f) ? 0.0f : __fdiv_rn(1.0f, scale);         // q4_0.rs:36
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            int j = w * 4 + b;
            int lo = sat_i8(__fadd_rn(product(v[j], r), 8.5f));
            int hi = sat_i8(__fadd_rn(product(v[j + 16], r), 8.5f));
            lo = lo < 15 ? lo : 15;
            hi = hi < 15 ? hi : 15;
            uint32_t byte = ((uint32_t)lo & 0xffu) | (((uint32_t)hi << 4) & 0xffu);
            word |= (byte & 0xffu) << (8 * b);
        }
        codes[w] = word;
    }
    return f32_to_f16_bits(scale);
}

}  // namespace
}  // namespace trocm
