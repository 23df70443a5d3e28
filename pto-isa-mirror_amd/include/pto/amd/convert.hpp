// TCVT, TFILLPAD, TRESHAPE, TSYNC and Event<> of the PTO header layer on gfx950.
// Reference semantics: TCVT cpu/TCvt.hpp:163-251 (convert_value, saturation clamp) with the FP8 rounding constructor of
// cpu/MXTypes.hpp:95-170; TFILLPAD cpu/TFillPad.hpp:22-64 (dst = src inside src's valid region, the pad value outside,
// over the whole static extent) with the pad bit patterns of common/constants.hpp:304-560; TRESHAPE cpu/TReshape.hpp
// (the destination tile aliases the source's storage); TSYNC / Event common/pto_instr.hpp:86-101, common/event.hpp:361-427.
#pragma once
#include "instr.hpp"

namespace pto {

enum class RoundMode : uint8_t { CAST_NONE = 0, CAST_RINT = 1, CAST_ROUND = 2, CAST_FLOOR = 3, CAST_CEIL = 4, CAST_TRUNC = 5, CAST_ODD = 6 };
enum class SaturationMode : uint8_t { ON = 0, OFF = 1 };
enum class TFillPadMode : uint8_t { Normal = 0, InPlace = 1, Expand = 2 };

namespace amd {

// ---- element conversions ---------------------------------------------------------------------------------------------
template <typename T>
constexpr bool is_float_like = std::is_same_v<T, float> || std::is_same_v<T, double> || std::is_same_v<T, _Float16> || std::is_same_v<T, __bf16>;
template <typename T>
constexpr bool is_fp8 = std::is_same_v<T, float8_e4m3_t> || std::is_same_v<T, float8_e5m2_t>;

// the value of an element as a double (exact for every source type of this path)
template <typename S>
PTO_INST double to_f64(S v)
{
    if constexpr (std::is_same_v<S, float8_e4m3_t>)
        return (double)ptoamd::e4m3_to_f32(v.raw);
    else if constexpr (std::is_same_v<S, float8_e5m2_t>)
        return (double)ptoamd::e5m2_to_f32(v.raw);
    else
        return (double)v;
}

// applyRoundingToIntegral (cpu/TCvt.hpp:80-113)
PTO_INST double round_to_integral(double v, RoundMode mode)
{
    switch (mode) {
        case RoundMode::CAST_RINT: return rint(v);
        case RoundMode::CAST_ROUND: return round(v);
        case RoundMode::CAST_FLOOR: return floor(v);
        case RoundMode::CAST_CEIL: return ceil(v);
        case RoundMode::CAST_TRUNC: return trunc(v);
        case RoundMode::CAST_ODD: {
            const double f = floor(v), frac = v - f;
            if (frac > 0.5)
                return f + 1;
            if (frac < 0.5)
                return f;
            return ((long long)f & 1) ? f : f + 1;  // a tie goes to the odd neighbour
        }
        default: return v;
    }
}

// The rounding constructor of the FP8 types (cpu/MXTypes.hpp:95-170): scale the magnitude to an integer significand
// of the target binade (subnormals included), round it in the requested mode, carry, saturate or overflow.
template <typename D>
PTO_INST uint8_t fp8_encode_round(double v, RoundMode mode, SaturationMode sat)
{
    constexpr bool e4 = std::is_same_v<D, float8_e4m3_t>;
    constexpr int ms = e4 ? 3 : 2, bias = e4 ? 7 : 15, max_exponent = e4 ? 8 : 15;
    constexpr uint32_t max_code = e4 ? 0x7Eu : 0x7Bu, overflow_code = e4 ? 0x7Fu : 0x7Cu;
    constexpr double max_value = e4 ? 448.0 : 57344.0;
    const uint64_t bits = (uint64_t)__double_as_longlong(v);
    const uint32_t sign = (bits >> 63) ? 0x80u : 0u;
    const double mag = fabs(v);
    if (v != v)
        return (uint8_t)(sign | 0x7Fu);
    if (sat == SaturationMode::ON && mag >= max_value)
        return (uint8_t)(sign | max_code);
    if (mag == __builtin_inf())
        return (uint8_t)(sign | overflow_code);
    if (mag == 0)
        return (uint8_t)sign;
    const bool toward_zero = mode == RoundMode::CAST_TRUNC || (mode == RoundMode::CAST_FLOOR && !sign) || (mode == RoundMode::CAST_CEIL && sign);
    if (mag >= ldexp(1.0, max_exponent + 1))
        return (uint8_t)(sign | ((!e4 && toward_zero) ? max_code : overflow_code));
    int exponent;
    (void)frexp(mag, &exponent);
    exponent = exponent - 1 > 1 - bias ? exponent - 1 : 1 - bias;
    const double scaled = ldexp(mag, ms - exponent);
    uint32_t sig = (uint32_t)scaled;
    const double rem = scaled - (double)sig;
    switch (mode) {
        case RoundMode::CAST_ROUND: sig += rem >= 0.5; break;
        case RoundMode::CAST_FLOOR: sig += sign && rem != 0; break;
        case RoundMode::CAST_CEIL: sig += !sign && rem != 0; break;
        case RoundMode::CAST_TRUNC: break;
        default: sig += rem > 0.5 || (rem == 0.5 && (sig & 1u)); break;  // NONE and ODD round like RINT
    }
    if (sig == (2u << ms)) {
        sig >>= 1;
        ++exponent;
    }
    uint32_t code = sig < (1u << ms) ? sig : (((uint32_t)(exponent + bias) << ms) + sig - (1u << ms));
    if (code > max_code)
        code = (sat == SaturationMode::ON || (!e4 && toward_zero)) ? max_code : overflow_code;
    return (uint8_t)(sign | code);
}

// SafeLimits (cpu/TCvt.hpp:115-142)
template <typename T>
PTO_INST constexpr double limit_lowest()
{
    if constexpr (std::is_same_v<T, _Float16>)
        return -65504.0;
    else if constexpr (std::is_same_v<T, __bf16>)
        return -3.3895313892515355e38;
    else if constexpr (std::is_same_v<T, float>)
        return -3.4028234663852886e38;
    else if constexpr (std::is_same_v<T, double>)
        return -1.7976931348623157e308;
    else if constexpr (std::is_signed_v<T>)
        return -(double)(1ull << (8 * sizeof(T) - 1));
    else
        return 0.0;
}
template <typename T>
PTO_INST constexpr double limit_max()
{
    if constexpr (std::is_same_v<T, _Float16>)
        return 65504.0;
    else if constexpr (std::is_same_v<T, __bf16>)
        return 3.3895313892515355e38;
    else if constexpr (std::is_same_v<T, float>)
        return 3.4028234663852886e38;
    else if constexpr (std::is_same_v<T, double>)
        return 1.7976931348623157e308;
    else if constexpr (std::is_signed_v<T>)
        return (double)((1ull << (8 * sizeof(T) - 1)) - 1);
    else
        return (double)(T) ~(T)0;
}

// convert_value (cpu/TCvt.hpp:163-205) after the optional saturation clamp of TCvt_Impl (:207-230)
template <typename D, typename S>
PTO_INST D tcvt_element(S val, RoundMode mode, SaturationMode sat)
{
    static_assert(!is_packed4<S> && !is_packed4<D>, "TCVT of packed fp4 tiles is not implemented on this backend");
    if constexpr (is_fp8<D>) {
        static_assert(is_float_like<S>, "TCVT to an FP8 type takes a floating source");
        D out;
        out.raw = fp8_encode_round<D>((double)val, mode, sat);
        return out;
    } else {
        if (sat == SaturationMode::ON) {
            if constexpr (!is_fp8<S>) {  // clamp in the source type to the range both types can hold
                double d = to_f64(val);
                constexpr double lo = limit_lowest<S>() > limit_lowest<D>() ? limit_lowest<S>() : limit_lowest<D>();
                constexpr double hi = limit_max<S>() < limit_max<D>() ? limit_max<S>() : limit_max<D>();
                d = d < lo ? lo : (d > hi ? hi : d);  // (a NaN passes through both comparisons)
                val = static_cast<S>(d);
            }
        }
        if constexpr (is_fp8<S>) {
            return static_cast<D>(to_f64(val));
        } else if constexpr (is_float_like<S> && std::is_integral_v<D>) {
            const double d = round_to_integral((double)val, mode);
            if constexpr (std::is_same_v<D, uint8_t>)
                return static_cast<D>(static_cast<int64_t>(d));
            else
                return static_cast<D>(d);
        } else if constexpr (std::is_integral_v<S> && is_float_like<D>) {
            return static_cast<D>(static_cast<double>(val));
        } else {
            return static_cast<D>(val);  // float-like to float-like: the compiler's conversion, round to nearest even
        }
    }
}

template <typename T, PadValue P>
PTO_INST T pad_element()
{
    if constexpr (!is_number<T>) {
        static_assert(P == PadValue::Zero || P == PadValue::Null, "one-byte code types pad with zero on this backend");
        return T{};
    } else if constexpr (P == PadValue::Max) {
        if constexpr (std::is_integral_v<T>)
            return std::is_signed_v<T> ? (T)((1ull << (8 * sizeof(T) - 1)) - 1) : (T)~(T)0;
        else
            return static_cast<T>(__builtin_inff());
    } else if constexpr (P == PadValue::Min) {
        if constexpr (std::is_integral_v<T>)
            return std::is_signed_v<T> ? (T)(1ull << (8 * sizeof(T) - 1)) : (T)0;
        else
            return static_cast<T>(-__builtin_inff());
    } else {
        return T(0);
    }
}

template <PadValue P, typename DstTile, typename SrcTile>
PTO_INST void tfillpad_lds(DstTile& dst, SrcTile& src)
{
    using T = typename DstTile::DType;
    static_assert(sizeof(T) == sizeof(typename SrcTile::DType), "TFILLPAD: source and destination element sizes differ");
    static_assert(DstTile::Loc != TileType::Acc && SrcTile::Loc != TileType::Acc, "TFILLPAD works on on-chip buffer tiles");
    static_assert(!is_packed4<T> || P == PadValue::Zero || P == PadValue::Null, "packed fp4 tiles pad with zero");
    if (dst.GetValidRow() == 0 || dst.GetValidCol() == 0)
        return;
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const uint8_t* s = src.Storage();
    uint8_t* d = dst.Storage();
    const bool in_place = s == d;
    __syncthreads();
    if constexpr (is_packed4<T>) {
        // two codes per byte, neighbours along a row or down a column (each tile says which); a thread builds one
        // destination byte from the two codes it holds, zero where the source has no valid element
        auto code = [&](int r, int c) -> uint32_t {
            if (r < vr && c < vc)
                return (s[src.ByteOffset(r, c)] >> (4 * SrcTile::Nibble(r, c))) & 0xFu;
            return 0u;
        };
        for (int idx = threadIdx.x; idx < DstTile::Rows * DstTile::Cols / 2; idx += PTO_AMD_THREADS) {
            int r, c;
            uint32_t lo, hi;
            if constexpr (DstTile::PairsDownColumns) {
                r = 2 * (idx / DstTile::Cols), c = idx - (r / 2) * DstTile::Cols;
                lo = code(r, c), hi = code(r + 1, c);
            } else {
                r = idx / (DstTile::Cols / 2), c = 2 * (idx - r * (DstTile::Cols / 2));
                lo = code(r, c), hi = code(r, c + 1);
            }
            d[dst.ByteOffset(r, c)] = (uint8_t)(lo | (hi << 4));
        }
    } else {
        const T pad = pad_element<T, P>();
        for (int idx = threadIdx.x; idx < DstTile::Rows * DstTile::Cols; idx += PTO_AMD_THREADS) {
            const int r = idx / DstTile::Cols, c = idx - r * DstTile::Cols;
            const bool inside = r < vr && c < vc;
            if (inside && in_place)
                continue;
            T v = pad;
            if (inside)
                v = *reinterpret_cast<const T*>(s + src.ByteOffset(r, c));
            *reinterpret_cast<T*>(d + dst.ByteOffset(r, c)) = v;
        }
    }
    __syncthreads();
}

}  // namespace amd

// ---- TCVT ------------------------------------------------------------------------------------------------------------
template <bool NeedSetCtrl = true, typename TileDataD, typename TileDataS, typename... WaitEvents>
PTO_INST RecordEvent TCVT(TileDataD& dst, TileDataS& src, RoundMode mode, SaturationMode satMode, WaitEvents&...)
{
    using D = typename TileDataD::DType;
    using S = typename TileDataS::DType;
    static_assert(TileDataD::Loc != TileType::Acc && TileDataS::Loc != TileType::Acc, "TCVT works on on-chip buffer tiles");
    PTO_AMD_TRACE_INSTR(1, TR_TCVT, dst, src);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const uint8_t* s = src.Storage();
    uint8_t* d = dst.Storage();
    __syncthreads();
    for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
        const int r = idx / vc, c = idx - r * vc;
        const S v = *reinterpret_cast<const S*>(s + src.ByteOffset(r, c));
        *reinterpret_cast<D*>(d + dst.ByteOffset(r, c)) = amd::tcvt_element<D, S>(v, mode, satMode);
    }
    __syncthreads();
    return {};
}
template <bool NeedSetCtrl = true, typename TileDataD, typename TileDataS, typename... WaitEvents>
PTO_INST RecordEvent TCVT(TileDataD& dst, TileDataS& src, RoundMode mode, WaitEvents&...)
{
    return TCVT<NeedSetCtrl>(dst, src, mode, SaturationMode::OFF);
}
template <bool NeedSetCtrl = true, typename TileDataD, typename TileDataS, typename TmpTileData, typename... WaitEvents,
          typename = std::enable_if_t<is_tile_data_v<TmpTileData>>>
PTO_INST RecordEvent TCVT(TileDataD& dst, TileDataS& src, TmpTileData&, RoundMode mode, SaturationMode satMode, WaitEvents&...)
{
    return TCVT<NeedSetCtrl>(dst, src, mode, satMode);
}
template <bool NeedSetCtrl = true, typename TileDataD, typename TileDataS, typename TmpTileData, typename... WaitEvents,
          typename = std::enable_if_t<is_tile_data_v<TmpTileData>>>
PTO_INST RecordEvent TCVT(TileDataD& dst, TileDataS& src, TmpTileData&, RoundMode mode, WaitEvents&...)
{
    return TCVT<NeedSetCtrl>(dst, src, mode, SaturationMode::OFF);
}

// ---- TFILLPAD --------------------------------------------------------------------------------------------------------
// Mat tile onto itself (or another tile of the same type): the pad value is a template argument, zero by default
// (reference: common/pto_instr.hpp:1612-1621)
template <typename TileData, PadValue PadVal = PadValue::Zero, std::enable_if_t<(TileData::Loc == TileType::Mat), int> = 0,
          typename... WaitEvents>
PTO_INST RecordEvent TFILLPAD(TileData& dst, TileData& src, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TFILLPAD, dst, src);
    amd::tfillpad_lds<PadVal>(dst, src);
    return {};
}
// Vec tiles: the destination tile's own PadVal (reference: common/pto_instr.hpp:1623-1653)
template <TFillPadMode mode = TFillPadMode::Normal, typename DstTileData, typename SrcTileData,
          std::enable_if_t<(DstTileData::Loc == TileType::Vec) && (SrcTileData::Loc == TileType::Vec), int> = 0, typename... WaitEvents>
PTO_INST RecordEvent TFILLPAD(DstTileData& dst, SrcTileData& src, WaitEvents&...)
{
    static_assert(DstTileData::PadVal != PadValue::Null, "TFILLPAD: the destination Vec tile needs a pad value");
    if constexpr (mode == TFillPadMode::Expand)
        static_assert(DstTileData::Cols >= SrcTileData::Cols && DstTileData::Rows >= SrcTileData::Rows, "TFILLPAD_EXPAND: the destination is at least as large as the source");
    else
        static_assert(DstTileData::Cols == SrcTileData::Cols && DstTileData::Rows == SrcTileData::Rows, "TFILLPAD: source and destination have the same static shape");
    PTO_AMD_TRACE_INSTR(1, TR_TFILLPAD, dst, src);
    amd::tfillpad_lds<DstTileData::PadVal>(dst, src);
    return {};
}
template <typename DstTileData, typename SrcTileData, typename... WaitEvents>
PTO_INST RecordEvent TFILLPAD_INPLACE(DstTileData& dst, SrcTileData& src, WaitEvents&... events)
{
    return TFILLPAD<TFillPadMode::InPlace>(dst, src, events...);
}
template <typename DstTileData, typename SrcTileData, typename... WaitEvents>
PTO_INST RecordEvent TFILLPAD_EXPAND(DstTileData& dst, SrcTileData& src, WaitEvents&... events)
{
    return TFILLPAD<TFillPadMode::Expand>(dst, src, events...);
}

// ---- TRESHAPE: the destination aliases the source's storage under another shape ---------------------------------------
template <typename TileDataOut, typename TileDataIn, typename... WaitEvents>
PTO_INST RecordEvent TRESHAPE(TileDataOut& dst, TileDataIn& src, WaitEvents&...)
{
    static_assert(TileDataIn::Loc == TileDataOut::Loc, "TRESHAPE: source and destination tile types differ");
    static_assert(TileDataIn::Bytes == TileDataOut::Bytes, "TRESHAPE: total byte size must match");
    static_assert((TileDataIn::SFractal == SLayout::NoneBox) == (TileDataOut::SFractal == SLayout::NoneBox),
                  "TRESHAPE: cannot reshape between boxed and non-boxed layouts");
    static_assert(TileDataIn::Loc != TileType::Acc && TileDataIn::Loc != TileType::Left && TileDataIn::Loc != TileType::Right,
                  "TRESHAPE works on row-major on-chip buffer tiles (Mat / Vec / Bias / Scaling) on this backend");
    PTO_AMD_TRACE_INSTR(1, TR_TRESHAPE, dst, src);
    dst.lds_ = src.lds_;
    dst.addr_ = src.addr_;
    dst.pend_ = src.pend_;
    return {};
}

// ---- TSYNC / Event ---------------------------------------------------------------------------------------------------
template <Op OpCode>
PTO_INST void TSYNC()
{
    __syncthreads();
}
template <typename... WaitEvents>
PTO_INST void TSYNC(WaitEvents&...)
{
    __syncthreads();
}

}  // namespace pto
