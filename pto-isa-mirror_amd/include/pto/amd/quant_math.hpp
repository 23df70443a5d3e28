// Scalar arithmetic of TQUANT's MX forms, bit-identical to the reference CPU simulator (include/pto/cpu/TQuant.hpp);
// shared by the streaming kernels behind the C ABI and by the tile instructions of the PTO header layer.
#pragma once
#include "device_types.hpp"

namespace ptoamd {

// shared-exponent algorithm x destination format (reference: MxQuantAlg, common/type.hpp:213-219)
enum { MX_OCP_FP8 = 0, MX_NV_FP8 = 1, MX_OCP_FP4 = 2, MX_NV_FP4 = 3 };

// ---- scalar pieces (TQuant.hpp:118-252) ---------------------------------------------------------------------

// EncodeE4M3Fn (TQuant.hpp:118-153): nearest finite E4M3 code to clamp(v, +-448), ties to the even code, and a result
// of zero is always code 0x00.  NV flushes |v| < 2^-10 to a signed zero first.
template <bool NV>
__device__ __forceinline__ uint32_t encode_e4m3fn(float v)
{
    const uint32_t vb = f2u(v);
    if ((vb & 0x7FFFFFFFu) > 0x7F800000u)
        return 0x7Fu;
    const uint32_t ab0 = vb & 0x7FFFFFFFu;
    if (NV && ab0 < 0x3A800000u /* 2^-10 */)
        return (vb >> 31) ? 0x80u : 0x00u;
    const uint32_t ab = ab0 > 0x43E00000u /* 448 */ ? 0x43E00000u : ab0;
    uint32_t code;
    if (ab < 0x3C800000u /* 2^-6: subnormal codes, step 2^-9 */) {
        code = (uint32_t)__float2int_rn(u2f(ab) * 512.0f);
    } else {
        const uint32_t r = ab + 0x7FFFFu + ((ab >> 20) & 1u);  // keep 3 mantissa bits, round to nearest even
        code = (r >> 20) - (120u << 3);
    }
    if (code == 0)
        return 0;
    return ((vb >> 31) << 7) | code;
}

// EncodeE2M1Magic (TQuant.hpp:155-176)
__device__ __forceinline__ uint32_t encode_e2m1_magic(float v)
{
    const uint32_t vb = f2u(v);
    const uint32_t ab = vb & 0x7FFFFFFFu;
    if (ab > 0x7F800000u)
        return 0x7u;
    const uint32_t sign = (vb >> 28) & 0x8u;
    if (ab == 0x7F800000u)
        return sign | 0x7u;
    uint32_t be = ab >> 23;
    be = be < 127u ? 127u : (be > 129u ? 129u : be);
    const uint32_t magic = (be + 22u) << 23;
    const uint32_t q = f2u(__fadd_rn(u2f(ab), u2f(magic))) - magic;
    const uint32_t mag = q + ((be - 127u) << 1);
    return sign | (mag < 7u ? mag : 7u);
}

// ComputeSharedExponent / ComputeE2M1SharedExponent / ComputeNvSharedExponent (TQuant.hpp:178-222)
template <int ALG>
__device__ __forceinline__ uint32_t shared_exponent(float maxabs)
{
    const uint32_t bits = f2u(maxabs);
    if (ALG == MX_OCP_FP8 || ALG == MX_OCP_FP4) {
        const uint32_t e = (bits & 0x7F800000u) >> 23, mant = bits & 0x7FFFFFu;
        const uint32_t sub = ALG == MX_OCP_FP8 ? 8u : 2u;
        if (e == 0xFFu && mant != 0)
            return 0xFFu;
        return e <= sub ? 0u : e - sub;
    }
    if (maxabs == 0.0f)
        return 0;
    const float descale = __fmul_rn(maxabs, ALG == MX_NV_FP8 ? (1.0f / 448.0f) : (1.0f / 6.0f));
    const uint32_t db = f2u(descale);
    const uint32_t e = (db & 0x7F800000u) >> 23, mant = db & 0x7FFFFFu;
    if (e == 0xFFu)
        return mant == 0 ? 0xFEu : 0xFFu;
    const bool up = mant > 0 && e != 0xFEu && !(e == 0 && mant <= 0x00400000u);
    return (e + (up ? 1u : 0u)) & 0xFFu;
}

// ComputeMxGroupScaling (TQuant.hpp:226-252, 336-347)
template <int ALG>
__device__ __forceinline__ float group_scaling(float maxabs, uint32_t e8m0)
{
    if (e8m0 == 0xFFu)
        return maxabs;
    if ((ALG == MX_NV_FP8 || ALG == MX_NV_FP4) && e8m0 == 0xFEu)
        return u2f(0x00400000u);  // 2^-127
    const uint32_t b = (254u - e8m0) << 23;
    return b == 0 ? u2f(0x00400000u) : u2f(b);
}

// ComputeMxGroupMax's per-element step (TQuant.hpp:280-306).  The running value is kept as bits: for OCP-FP4 it is
// the maximum of truncated-bf16 magnitude patterns, otherwise max(fabs) where NaN never wins.  NV-FP4 returns the first
// NaN of the group as it stands (sign and payload): a NaN at position pos (0 .. 31 in group order) is carried as
// bit 31 | (31 - pos) << 26 | sign << 23 | mantissa, which is larger than every magnitude pattern and larger for an
// earlier position, so one unsigned max over the group -- in any order, across lanes -- leaves the first NaN.
template <int ALG>
__device__ __forceinline__ uint32_t max_step(uint32_t run, float v, int pos = 0)
{
    const uint32_t ab = f2u(v) & 0x7FFFFFFFu;
    if (ALG == MX_OCP_FP4) {
        const uint32_t t = ab & 0x7FFF0000u;
        return t > run ? t : run;
    }
    if (ab > 0x7F800000u) {  // NaN
        if (ALG != MX_NV_FP4)
            return run;
        const uint32_t tag = 0x80000000u | ((uint32_t)(31 - pos) << 26) | ((f2u(v) >> 31) << 23) | (ab & 0x007FFFFFu);
        return tag > run ? tag : run;
    }
    return ab > run ? ab : run;
}
template <int ALG>
__device__ __forceinline__ uint32_t max_merge(uint32_t a, uint32_t b)
{
    return a > b ? a : b;  // bit patterns of non-negative floats order like the floats; a tagged NaN is larger than all
}
template <int ALG>
__device__ __forceinline__ float max_value(uint32_t run)
{
    if (ALG == MX_NV_FP4 && (run >> 31))
        return u2f(0x7F800000u | ((run & 0x00800000u) << 8) | (run & 0x007FFFFFu));
    return u2f(run);
}

template <typename T>
__device__ __forceinline__ float widen(T v);
template <>
__device__ __forceinline__ float widen<float>(float v) { return v; }
struct half_bits { uint16_t b; };
struct bf16_bits { uint16_t b; };
template <>
__device__ __forceinline__ float widen<half_bits>(half_bits v) { return f16_bits_to_f32(v.b); }
template <>
__device__ __forceinline__ float widen<bf16_bits>(bf16_bits v) { return bf16_bits_to_f32(v.b); }

// StoreMxEncodedValue (TQuant.hpp:349-372)
template <int ALG, bool SRC_BF16>
__device__ __forceinline__ uint32_t encode_mx(float v, float scaling)
{
    if (ALG == MX_OCP_FP8 || ALG == MX_NV_FP8)
        return encode_e4m3fn<ALG == MX_NV_FP8>(__fmul_rn(v, scaling));
    const uint32_t sb = f2u(scaling);
    if ((sb & 0x7FFFFFFFu) == 0x7F800000u)
        return (sb >> 31) ? 0xFu : 0x7u;
    if ((sb & 0x7FFFFFFFu) > 0x7F800000u)
        return 0x7u;
    float scaled = __fmul_rn(v, scaling);
    if (SRC_BF16)  // bf16 sources re-round the scaled value to bf16 (TQuant.hpp:68-76)
        scaled = bf16_bits_to_f32(f32_to_bf16_bits(scaled));
    return encode_e2m1_magic(scaled);
}

}  // namespace ptoamd
