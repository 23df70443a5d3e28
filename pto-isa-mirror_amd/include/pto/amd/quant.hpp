// TQUANT and TDEQUANT on LDS-resident tiles.  Reference semantics: cpu/TQuant.hpp:78-96,461-547 (INT8 forms, MX forms
// with 32-element groups along a row), cpu/TDeQuant.hpp:18-37; wrapper signatures common/pto_instr.hpp:2978-3072.
// The scalar arithmetic is quant_math.hpp's, shared with the streaming kernels behind the C ABI, so codes, exponents,
// group maxima and scalings are bit-identical to the simulator's.
#pragma once
#include "quant_math.hpp"
#include "tile.hpp"

namespace pto {

enum class QuantType { MXFP8 = 0, MXFP4_E2M1 = 1, INT8_SYM = 2, INT8_ASYM = 3 };
enum class QuantScaleAlg { OCP = 0, NV = 1 };
enum class MxQuantAlg { OcpMxFp8E4M3 = 0, NvMxFp8E4M3 = 1, OcpMxFp4E2M1 = 2, NvMxFp4E2M1 = 3 };
enum class VecStoreMode { ND = 0, NZ = 1 };

namespace amd {

template <typename T>
PTO_INST float to_float(T v)
{
    return static_cast<float>(v);
}
// parameter tiles are read with the row / column clamped to their valid extent (reference: cpu/TQuant.hpp:78-84)
template <typename TilePara>
PTO_INST float para(const TilePara& t, int r, int c)
{
    const int rr = min(r, max(t.GetValidRow(), 1) - 1), cc = min(c, max(t.GetValidCol(), 1) - 1);
    return to_float(*reinterpret_cast<const typename TilePara::DType*>(t.Storage() + t.ByteOffset(rr, cc)));
}

template <bool ASYM, typename TileOut, typename TileSrc, typename TilePara>
PTO_INST void tquant_int8(TileOut& dst, TileSrc& src, TilePara& scale, TilePara* offset)
{
    static_assert(std::is_same_v<typename TileSrc::DType, float>, "TQUANT INT8 takes a float source tile");
    static_assert(sizeof(typename TileOut::DType) == 1, "TQUANT INT8 writes one byte per element");
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    __syncthreads();
    for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
        const int r = idx / vc, c = idx - r * vc;
        float v = __fmul_rn(*reinterpret_cast<const float*>(src.Storage() + src.ByteOffset(r, c)), para(scale, r, c));
        if constexpr (ASYM)
            v = __fadd_rn(v, para(*offset, r, c));
        v = rintf(v);
        const float lo = ASYM ? 0.0f : -128.0f, hi = ASYM ? 255.0f : 127.0f;
        v = v < lo ? lo : (v > hi ? hi : v);
        *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(r, c)) = (uint8_t)(int)v;
    }
    __syncthreads();
}

// one thread per 32-element group along a row
template <int ALG, typename TileOut, typename TileSrc, typename TileExp, typename TileMax, typename TileScaling>
PTO_INST void tquant_mx(TileOut& dst, TileSrc& src, TileExp* exp, TileMax* mx, TileScaling* scaling)
{
    using S = typename TileSrc::DType;
    constexpr bool SRC_BF16 = std::is_same_v<S, __bf16>;
    constexpr bool FP4 = ALG == ptoamd::MX_OCP_FP4 || ALG == ptoamd::MX_NV_FP4;
    static_assert(std::is_same_v<S, float> || std::is_same_v<S, _Float16> || SRC_BF16, "TQUANT MX: source is float, half or bf16");
    const int vr = src.GetValidRow(), vc = src.GetValidCol(), groups_per_row = vc / 32;
    __syncthreads();
    for (int g = threadIdx.x; g < vr * groups_per_row; g += PTO_AMD_THREADS) {
        const int r = g / groups_per_row, c0 = (g - r * groups_per_row) * 32;
        uint32_t run = 0;
        for (int i = 0; i < 32; ++i)
            run = ptoamd::max_step<ALG>(run, to_float(*reinterpret_cast<const S*>(src.Storage() + src.ByteOffset(r, c0 + i))), i);
        const float maxabs = ptoamd::max_value<ALG>(run);
        const uint32_t e = ptoamd::shared_exponent<ALG>(maxabs);
        const float sc = ptoamd::group_scaling<ALG>(maxabs, e);
        if (exp)
            *reinterpret_cast<uint8_t*>(exp->Storage() + g) = (uint8_t)e;
        if (mx)
            reinterpret_cast<float*>(mx->Storage())[g] = maxabs;
        if (scaling)
            reinterpret_cast<float*>(scaling->Storage())[g] = sc;
        for (int i = 0; i < 32; i += 2) {
            const float v0 = to_float(*reinterpret_cast<const S*>(src.Storage() + src.ByteOffset(r, c0 + i)));
            const float v1 = to_float(*reinterpret_cast<const S*>(src.Storage() + src.ByteOffset(r, c0 + i + 1)));
            const uint32_t q0 = ptoamd::encode_mx<ALG, SRC_BF16>(v0, sc), q1 = ptoamd::encode_mx<ALG, SRC_BF16>(v1, sc);
            if constexpr (FP4) {
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(r, c0 + i)) = (uint8_t)(q0 | (q1 << 4));
            } else {
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(r, c0 + i)) = (uint8_t)q0;
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(r, c0 + i + 1)) = (uint8_t)q1;
            }
        }
    }
    __syncthreads();
}

// groups of 32 along a column (grouping axis 0, the DN form): one thread per (group, column pair); exp / max / scaling
// are [rows / 32][cols]
template <int ALG, typename TileOut, typename TileSrc, typename TileExp, typename TileMax, typename TileScaling>
PTO_INST void tquant_mx_cols(TileOut& dst, TileSrc& src, TileExp* exp, TileMax* mx, TileScaling* scaling)
{
    using S = typename TileSrc::DType;
    constexpr bool SRC_BF16 = std::is_same_v<S, __bf16>;
    constexpr bool FP4 = ALG == ptoamd::MX_OCP_FP4 || ALG == ptoamd::MX_NV_FP4;
    const int vr = src.GetValidRow(), vc = src.GetValidCol(), groups = vr / 32, pairs = vc / 2;
    auto at = [&](int r, int c) { return to_float(*reinterpret_cast<const S*>(src.Storage() + src.ByteOffset(r, c))); };
    __syncthreads();
    for (int idx = threadIdx.x; idx < groups * pairs; idx += PTO_AMD_THREADS) {
        const int g = idx / pairs, c0 = 2 * (idx - g * pairs);
        float sc[2];
        for (int j = 0; j < 2; ++j) {
            uint32_t run = 0;
            for (int r = 0; r < 32; ++r)
                run = ptoamd::max_step<ALG>(run, at(g * 32 + r, c0 + j), r);
            const float maxabs = ptoamd::max_value<ALG>(run);
            const uint32_t e = ptoamd::shared_exponent<ALG>(maxabs);
            sc[j] = ptoamd::group_scaling<ALG>(maxabs, e);
            const int gi = g * vc + c0 + j;
            if (exp)
                *reinterpret_cast<uint8_t*>(exp->Storage() + gi) = (uint8_t)e;
            if (mx)
                reinterpret_cast<float*>(mx->Storage())[gi] = maxabs;
            if (scaling)
                reinterpret_cast<float*>(scaling->Storage())[gi] = sc[j];
        }
        for (int r = 0; r < 32; ++r) {
            const int row = g * 32 + r;
            const uint32_t q0 = ptoamd::encode_mx<ALG, SRC_BF16>(at(row, c0), sc[0]);
            const uint32_t q1 = ptoamd::encode_mx<ALG, SRC_BF16>(at(row, c0 + 1), sc[1]);
            if constexpr (FP4) {
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(row, c0)) = (uint8_t)(q0 | (q1 << 4));
            } else {
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(row, c0)) = (uint8_t)q0;
                *reinterpret_cast<uint8_t*>(dst.Storage() + dst.ByteOffset(row, c0 + 1)) = (uint8_t)q1;
            }
        }
    }
    __syncthreads();
}

}  // namespace amd

// INT8: dst = clamp(nearbyint(src * scale[row] (+ offset[row]))); the "scale" operand multiplies
template <auto quant_type, typename TileDataOut, typename TileDataSrc, typename TileDataPara,
          typename = std::enable_if_t<quant_type == QuantType::INT8_SYM || quant_type == QuantType::INT8_ASYM>>
PTO_INST RecordEvent TQUANT(TileDataOut& dst, TileDataSrc& src, TileDataPara& scale, TileDataPara* offset = nullptr)
{
    PTO_AMD_TRACE_INSTR(1, TR_TQUANT, dst, src, scale);
    amd::tquant_int8<quant_type == QuantType::INT8_ASYM>(dst, src, scale, offset);
    return {};
}

// MX: dst codes (E4M3 bytes or packed E2M1 pairs), exp [rows][cols / 32] E8M0, max and scaling per group (flat)
template <auto quant_type, typename TileDataOut, typename TileDataSrc, typename TileDataExp, typename TileDataMax,
          typename TileDataScaling, auto scale_alg = QuantScaleAlg::OCP,
          typename = std::enable_if_t<quant_type == QuantType::MXFP8 || quant_type == QuantType::MXFP4_E2M1>>
PTO_INST RecordEvent TQUANT(TileDataOut& dst, TileDataSrc& src, TileDataExp* exp, TileDataMax* max, TileDataScaling* scaling)
{
    constexpr int alg = (quant_type == QuantType::MXFP8 ? 0 : 2) + (scale_alg == QuantScaleAlg::NV ? 1 : 0);
    PTO_AMD_TRACE_INSTR(1, TR_TQUANT, dst, src);
    amd::tquant_mx<alg>(dst, src, exp, max, scaling);
    return {};
}

// MXFP8, NZ store mode: as above, and the exponents once more in exp_zz in the order of 16-row x 2-group boxes (the
// layout of an MX matmul's left scale tile): box (row / 16, group / 2), then row % 16, then group % 2
// (reference: cpu/TQuant.hpp:254-278, 585-611)
template <auto quant_type, auto store_mode, typename TileDataOut, typename TileDataSrc, typename TileDataExp,
          typename TileDataMax, typename TileDataScaling,
          typename = std::enable_if_t<std::is_same_v<decltype(store_mode), VecStoreMode>>>
PTO_INST RecordEvent TQUANT(TileDataOut& dst, TileDataSrc& src, TileDataExp* exp, TileDataMax* max, TileDataScaling* scaling,
                            TileDataExp* exp_zz)
{
    static_assert(quant_type == QuantType::MXFP8, "TQUANT: the NZ store mode is defined for MXFP8");
    static_assert(store_mode == VecStoreMode::NZ, "TQUANT: this overload is the NZ store mode");
    PTO_AMD_TRACE_INSTR(1, TR_TQUANT, dst, src);
    amd::tquant_mx<0>(dst, src, exp, max, scaling);
    const int rows = src.GetValidRow(), groups = src.GetValidCol() / 32;
    if (exp == nullptr || exp_zz == nullptr || rows % 16 != 0 || groups % 2 != 0) {
        amd::report(2);  // the reorder needs whole 16 x 2 boxes
        return {};
    }
    for (int i = threadIdx.x; i < rows * groups; i += PTO_AMD_THREADS) {
        const int r = i / groups, g = i - r * groups;
        const int zz = ((r / 16) * (groups / 2) + g / 2) * 32 + (r % 16) * 2 + g % 2;
        *reinterpret_cast<uint8_t*>(exp_zz->Storage() + zz) = *reinterpret_cast<const uint8_t*>(exp->Storage() + i);
    }
    __syncthreads();
    return {};
}

// MX with an explicit grouping axis (1: along a row, 0: along a column) and the unified algorithm tag
// (reference: common/pto_instr.hpp:3006-3019, cpu/TQuant.hpp:524-547)
template <int grp_axis, auto mx_alg, typename TileDataOut, typename TileDataSrc, typename TileDataExp, typename TileDataMax,
          typename TileDataScaling>
PTO_INST RecordEvent TQUANT(TileDataOut& dst, TileDataSrc& src, TileDataExp* exp, TileDataMax* max, TileDataScaling* scaling)
{
    static_assert(grp_axis == 0 || grp_axis == 1, "TQUANT: the grouping axis is 0 or 1");
    static_assert(std::is_same_v<decltype(mx_alg), MxQuantAlg>, "TQUANT<grp_axis, mx_alg>: mx_alg is an MxQuantAlg");
    constexpr int alg = static_cast<int>(mx_alg);
    static_assert(alg >= 0 && alg <= 3, "TQUANT: the HiFloat4 algorithm is not implemented on this backend");
    PTO_AMD_TRACE_INSTR(1, TR_TQUANT, dst, src);
    if constexpr (grp_axis == 1)
        amd::tquant_mx<alg>(dst, src, exp, max, scaling);
    else
        amd::tquant_mx_cols<alg>(dst, src, exp, max, scaling);
    return {};
}

// dst(r, c) = (D(src(r, c)) - D(offset(r, pc))) * D(scale(r, pc)), pc = min(c, max(1, scale.validCol) - 1)
template <typename TileDataDst, typename TileDataSrc, typename TileDataPara, typename... WaitEvents>
PTO_INST RecordEvent TDEQUANT(TileDataDst& dst, TileDataSrc& src, TileDataPara& scale, TileDataPara& offset, WaitEvents&...)
{
    using D = typename TileDataDst::DType;
    static_assert(std::is_same_v<D, float>, "TDEQUANT writes a float tile on this backend");
    PTO_AMD_TRACE_INSTR(1, TR_TDEQUANT, dst, src, scale, offset);
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    __syncthreads();
    for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
        const int r = idx / vc, c = idx - r * vc;
        const int pc = min(c, max(1, scale.GetValidCol()) - 1);
        const float s = amd::to_float(*reinterpret_cast<const typename TileDataPara::DType*>(scale.Storage() + scale.ByteOffset(r, pc)));
        const float o = amd::to_float(*reinterpret_cast<const typename TileDataPara::DType*>(offset.Storage() + offset.ByteOffset(r, pc)));
        const float v = amd::to_float(*reinterpret_cast<const typename TileDataSrc::DType*>(src.Storage() + src.ByteOffset(r, c)));
        *reinterpret_cast<float*>(dst.Storage() + dst.ByteOffset(r, c)) = __fmul_rn(__fsub_rn(v, o), s);
    }
    __syncthreads();
    return {};
}

}  // namespace pto
