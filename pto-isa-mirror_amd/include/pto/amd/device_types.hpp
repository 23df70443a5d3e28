// Device-side element types and conversions for the gfx950 backend.
// Semantics follow the reference CPU simulator's types (include/pto/cpu/MXTypes.hpp:232-274 for the MX decode,
// include/pto/cpu/TQuant.hpp:49-55 for bf16 rounding); the static_cast<half> of TSTORE is IEEE round-to-nearest-even.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ptoamd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) int i32x16;

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// float -> bf16 bits, round to nearest even; NaN keeps a quiet payload
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f)
{
    const uint32_t b = f2u(f);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((b >> 16) | 0x0040u);
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
// two floats -> two bf16 in one dword (a in the low half): v_cvt_pk_bf16_f32, round to nearest even, NaNs stay quiet NaNs
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float a, float b)
{
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// float -> fp16 bits, round to nearest even (v_cvt_f16_f32 under the default rounding mode)
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f)
{
    const _Float16 h = (_Float16)f;
    return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

// E8M0 -> 2^(e-127) as a double (e = 0 -> 2^-127, e = 255 -> 2^128, no NaN; MXTypes.hpp:254-259)
__device__ __forceinline__ double e8m0_to_f64(uint32_t e)
{
    return __longlong_as_double((long long)((uint64_t)(e + 1023u - 127u) << 52));
}
// E8M0 -> float scale; 2^-127 is a float denormal, 2^128 overflows to +inf
__device__ __forceinline__ float e8m0_to_f32(uint32_t e)
{
    return e == 0 ? u2f(0x00400000u) : u2f(e << 23);
}

// Fix-pipe quantisation words (reference: cpu/common.hpp:117-185).  A scalar word carries an fp32 scale in its low 32
// bits; a vector (per-column) word a 19-bit (1, 8, 10) float at bits 13..31.  Bits 37..45 hold the offset added before
// rounding to an 8-bit target and bit 46 that target's signedness.
template <bool VECTOR>
__device__ __forceinline__ float fixpipe_word_scale(uint64_t word)
{
    if (!VECTOR)
        return u2f((uint32_t)(word & 0xFFFFFFFFu));
    const uint32_t m1 = (uint32_t)((word >> 13) & 0x7FFFFu);
    const uint32_t s = (m1 >> 18) & 1u, e = (m1 >> 10) & 0xFFu, mant = m1 & 0x3FFu;
    if (e == 0 && mant == 0)
        return 0.0f;
    const float mv = 1.0f + (float)mant / 1024.0f;
    return __fmul_rn(__fmul_rn(s ? -1.0f : 1.0f, mv), e8m0_to_f32(e));
}
// acc * scale, then: 8-bit targets add the offset, round to nearest even and clamp to the signed or unsigned byte range
// (the result is the integer as a float); the half target clamps finite values to +-65504 (every value when the
// accumulator was an integer)
template <bool VECTOR, bool TO_BYTE, bool SRC_INT>
__device__ __forceinline__ float fixpipe_quantize(float acc, uint64_t word)
{
    float r = __fmul_rn(acc, fixpipe_word_scale<VECTOR>(word));
    if (TO_BYTE) {
        const float offset = (float)(uint32_t)((word >> 37) & 0x1FFu);
        const bool sign = (word >> 46) & 1u;
        const float rounded = rintf(__fadd_rn(r, offset));
        const float lo = sign ? -128.0f : 0.0f, hi = sign ? 127.0f : 255.0f;
        r = rounded < lo ? lo : (rounded > hi ? hi : rounded);
    } else if (SRC_INT || (r == r && fabsf(r) != __builtin_inff())) {
        r = r < -65504.0f ? -65504.0f : (r > 65504.0f ? 65504.0f : r);
    }
    return r;
}

// The fix-pipe's saturation control (bit 48 of the task cookie, cpu/common.hpp:146,157-171): with it set, the half and
// bfloat16 targets turn a NaN product into 0 and clamp an infinite one to the largest finite value of the target's
// range like any other (without it, non-finite products pass through).  `r` is acc * scale of a float accumulator.
template <bool TO_F16>
__device__ __forceinline__ float fixpipe_saturate_inf(float r)
{
    if (r != r)
        return 0.0f;
    const float hi = TO_F16 ? 65504.0f : 3.402823466e38f;
    return r < -hi ? -hi : (r > hi ? hi : r);
}

// the int16 shift mode of the fix-pipe (cpu/common.hpp:174-180): arithmetic shift right by bits 32..35 of the word plus
// one; the reference narrows to int16 before it clamps, so the value wraps
__device__ __forceinline__ int32_t fixpipe_shift_s16(int32_t acc, uint64_t word)
{
    return (int32_t)(int16_t)(acc >> ((int)((word >> 32) & 0xFu) + 1));
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t c)
{
    const uint32_t mag = c & 0x7Fu;
    if (mag == 0x7Fu)
        return u2f(0x7FC00000u | ((c & 0x80u) << 24));
    const uint32_t e = mag >> 3, m = mag & 7u;
    float v = e == 0 ? (float)m * 0.001953125f /* 2^-9 */ : u2f(((e + 120u) << 23) | (m << 20));
    return (c & 0x80u) ? -v : v;
}
__device__ __forceinline__ float e5m2_to_f32(uint32_t c)
{
    // E5M2 is the upper byte of an IEEE half
    return f16_bits_to_f32((uint16_t)(c << 8));
}
// HiFloat8 (reference: include/pto/cpu/Hifloat8.hpp:65-135): sign, then a prefix code that says how many of the remaining
// bits are exponent (4, 3, 2, 1 or 0; sign-magnitude with an implicit leading one) and how many mantissa (1, 2, 3, 3, 3);
// payloads 1 .. 7 are the powers of two 2^-22 .. 2^-16, 0x00 is zero, 0x80 NaN, 0x6F / 0xEF the infinities.  Every value is
// exact in float (and in bfloat16).
__device__ __forceinline__ float hif8_to_f32(uint32_t c)
{
    const uint32_t sign = (c & 0x80u) << 24, p = c & 0x7Fu;
    if ((p >> 3) == 0) {
        if (p == 0)
            return sign ? u2f(0x7FC00000u) : 0.0f;
        return u2f(sign | ((p + 104u) << 23));  // 2^(p - 23)
    }
    int ebits, mbits;
    if ((p >> 5) != 0) {
        ebits = (int)(p >> 5) + 1;  // prefixes 01, 10, 11 -> 2, 3, 4 exponent bits out of 5
        mbits = 5 - ebits;
    } else if ((p >> 4) == 1) {
        ebits = 1;
        mbits = 3;
    } else {
        ebits = 0;
        mbits = 3;
    }
    const uint32_t rest = p & ((1u << (ebits + mbits)) - 1u);
    const uint32_t raw_e = rest >> mbits, raw_m = rest & ((1u << mbits) - 1u);
    int e = 0;
    if (ebits > 0) {
        const uint32_t sbit = raw_e & (1u << (ebits - 1));
        const int mag = (int)((1u << (ebits - 1)) | (raw_e - sbit));
        e = sbit ? -mag : mag;
    }
    if (ebits == 4 && e == 15 && raw_m == 1)
        return u2f(sign | 0x7F800000u);
    return u2f(sign | ((uint32_t)(e + 127) << 23) | (raw_m << (23 - mbits)));
}
__device__ __forceinline__ float e2m1_to_f32(uint32_t c)
{
    const uint32_t mag = c & 7u;
    const uint32_t e = mag >> 1, m = mag & 1u;
    const float v = e == 0 ? 0.5f * (float)m : u2f(((e + 126u) << 23) | (m << 22));
    return (c & 8u) ? -v : v;  // code 0x8 gives -0, which contributes nothing to a sum (the reference decodes +0)
}
__device__ __forceinline__ float e1m2_to_f32(uint32_t c)
{
    const float v = 0.25f * (float)(c & 7u);  // e = 0: m/4; e = 1: (1 + m/4) = (4 + m)/4
    return (c & 8u) ? -v : v;
}

}  // namespace ptoamd
