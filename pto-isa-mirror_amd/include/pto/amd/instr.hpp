// The tile instructions of the matmul path as workgroup-collective device functions.
// Reference semantics: TLOAD cpu/TLoad.hpp:287-321; TMOV cpu/TMov.hpp:21-35; TEXTRACT cpu/TExtract.hpp:21-46;
// TMATMUL / _ACC / _BIAS / TGEMV* cpu/TMatmul.hpp:77-113,207-252; TSTORE cpu/TStore.hpp:41-79,
// cpu/common.hpp:187-198 (relu then static_cast).  Wrapper signatures: common/pto_instr.hpp:257-268,377-447,952-1010.
//
// Ordering: every instruction that writes LDS starts with a workgroup barrier (earlier readers of the bytes it overwrites
// are done) and ends with one, with one exception: a TLOAD that can run as LDS-DMA (a fully valid boxed Mat tile from a
// 16-byte aligned ND / DN global tensor) only issues its copies and marks the tile pending; the first instruction that
// reads the tile waits for the copies and for the other waves (acquire).  Between the TLOAD and that read the core is
// free to run other tile instructions -- the TMATMULs of the previous panel -- which is how a PTO program's
// double-buffered L1 panels overlap copy-in and MFMA on this backend.  Instructions that only read LDS need no barrier
// of their own.
#pragma once
#include <utility>

#include "device_types.hpp"
#include "lds_dma.hpp"
#include "tile.hpp"
#include "trace.hpp"

namespace pto {
namespace amd {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int i32x4v __attribute__((ext_vector_type(4)));
// staging accesses: one wave writes its band as register quads and reads it back as 16-byte row chunks with no workgroup
// barrier in between, so the two access types must be allowed to alias and the compiler may not move one across the other
typedef int i32x4s __attribute__((ext_vector_type(4), may_alias));
typedef int i32x2s __attribute__((ext_vector_type(2), may_alias));
typedef int i32x2v_plain __attribute__((ext_vector_type(2)));

template <typename D, typename S>
PTO_INST D convert(S v)
{
    return static_cast<D>(v);  // float -> _Float16 / __bf16: round to nearest even, as the reference's static_cast
}

// number of bytes one logical element occupies for plain (non-packed) types
template <typename T>
constexpr bool is_number = std::is_integral_v<T> || std::is_same_v<T, float> || std::is_same_v<T, double> ||
                           std::is_same_v<T, _Float16> || std::is_same_v<T, __bf16>;
template <typename T>
constexpr bool is_packed4 = std::is_same_v<T, float4_e2m1x2_t> || std::is_same_v<T, float4_e1m2x2_t>;

// a Mat tile whose asynchronous TLOAD may still be in flight: wait for this wave's copies, then for every wave's
template <typename TileData>
PTO_INST void acquire(TileData& t)
{
    if constexpr (TileData::Loc == TileType::Mat) {
        if (t.pend_) {  // the same value in every thread of the core
            dma_wait();
            __syncthreads();
            t.pend_ = 0;
        }
    }
}

// Several freshly loaded Mat tiles at once: one wait and one workgroup barrier for all of them, where acquiring them one
// by one (the first TEXTRACT / TMOV of each) brings a barrier per tile.
template <typename... Tiles>
PTO_INST void acquire_all(Tiles&... t)
{
    static_assert(((Tiles::Loc == TileType::Mat) && ...), "only Mat tiles are loaded asynchronously");
    if ((... || (t.pend_ != 0))) {  // the same value in every thread of the core
        dma_wait();
        __syncthreads();
        ((t.pend_ = 0), ...);
    }
}

// ---- TLOAD as LDS-DMA -------------------------------------------------------------------------------------------------
// A boxed Mat tile is stored as swizzled lines (rows for the A-side layouts, columns for the B-side ones).  When the
// global tensor delivers those lines contiguously -- ND for row lines, DN for column lines -- every 16-byte chunk of
// the tile is one lane of a global_load_lds_dwordx4: chunk position q of the tile's storage (line q / C, position
// q % C) is fetched from the line's logical chunk (q % C) ^ swizzle(line), because the DMA writes lanes linearly and the
// swizzle therefore has to be applied on the global side.  Returns false (nothing done) when the operands do not
// qualify; the caller then takes the element-wise path.
template <typename TileData, typename GlobalData>
PTO_INST bool tload_dma(TileData& dst, GlobalData& src)
{
    using T = typename TileData::DType;
    // (the E8M0 scale matrices: MX_A_ND keeps a row's K-groups contiguous like ND, MX_B_DN a column's like DN; their
    // shapes are (1, 1, lines, groups / 2, 2) with strides (., ., line pitch, 2, 1))
    constexpr bool nd = GlobalData::layout == Layout::ND, dn = GlobalData::layout == Layout::DN;
    constexpr bool mx_a = GlobalData::layout == Layout::MX_A_ND, mx_b = GlobalData::layout == Layout::MX_B_DN;
    if constexpr (TileData::MatLines && TileData::LineBytes % 16 == 0 && sizeof(T) == sizeof(typename GlobalData::DType) &&
                  (((nd || mx_a) && TileData::LinesAreRows) || ((dn || mx_b) && !TileData::LinesAreRows))) {
        // ND: element (r, c) at r * stride[3] + c * stride[4]; DN: the same with the unit stride on the rows
        const int64_t line_stride = src.GetStride((mx_a || mx_b) ? 2 : (nd ? 3 : 4));
        const int64_t gbytes = line_stride * (int64_t)ElemTraits<T>::bytes2 / 2;  // (packed fp4: strides count codes)
        const uintptr_t gaddr = reinterpret_cast<uintptr_t>(src.data());
        bool shape_ok;
        if constexpr (mx_a || mx_b)
            shape_ok = src.GetShape(0) == 1 && src.GetShape(1) == 1 && src.GetStride(3) == 2 && src.GetStride(4) == 1 &&
                       src.GetShape(4) == 2 && src.GetShape(2) >= TileData::Lines && src.GetShape(3) * 2 >= TileData::LineBytes;
        else
            shape_ok = src.GetShape(0) == 1 && src.GetShape(1) == 1 && src.GetShape(2) == 1 && src.GetStride(nd ? 4 : 3) == 1 &&
                       src.GetShape(3) >= TileData::Rows && src.GetShape(4) >= TileData::Cols;
        const bool ok = shape_ok && dst.GetValidRow() == TileData::Rows && dst.GetValidCol() == TileData::Cols && (gbytes & 15) == 0 &&
                        (gaddr & 15u) == 0 && gbytes > 0 &&
                        (int64_t)(TileData::Lines - 1) * gbytes + TileData::LineBytes <= (int64_t)0xFFFFFFFFll;
        if (!ok)
            return false;
        acquire(dst);     // an earlier asynchronous load of the same tile has landed before it is overwritten
#ifndef PTO_AMD_TLOAD_AFTER_ACQUIRE
        __syncthreads();  // earlier readers of the tile (TMATMULs through windows, TMOVs) are done
#endif
        constexpr int C = TileData::LineBytes / 16, total = TileData::Lines * C;
        constexpr int iters = (total + PTO_AMD_THREADS - 1) / PTO_AMD_THREADS;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t lds0 = lds_address_of(dst.Storage()) + wave * 1024u;
        const uint32_t gb32 = (uint32_t)gbytes;
#pragma unroll
        for (int i = 0; i < iters; ++i) {
            const uint32_t q = threadIdx.x + i * PTO_AMD_THREADS;
            if (total % PTO_AMD_THREADS == 0 || q < (uint32_t)total) {
                const uint32_t line = q / C, pos = q % C;
                const uint32_t chunk = pos ^ ((line >> TileData::Swz::sh) & TileData::Swz::mask);
                lds_dma16_off(reinterpret_cast<const uint8_t*>(src.data()), line * gb32 + chunk * 16u,
                              lds0 + (uint32_t)i * (PTO_AMD_THREADS * 16u));
            }
        }
        dst.pend_ = 1;
        return true;
    } else {
        return false;
    }
}

// ---- generic element movement between global memory and an LDS tile ------------------------------------------------
template <typename TileData, typename GlobalData>
PTO_INST void tload_lds(TileData& dst, GlobalData& src)
{
    using T = typename TileData::DType;
    static_assert(sizeof(T) == sizeof(typename GlobalData::DType), "TLOAD: tile and global element sizes differ");
    if (tload_dma(dst, src))
        return;
    acquire(dst);
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    const auto* g = reinterpret_cast<const T*>(src.data());
    uint8_t* base = dst.Storage();
    __syncthreads();
    if constexpr (is_packed4<T>) {
        // Two codes per byte.  In global memory the pair runs along the unit-stride direction (a row of an ND tensor, a
        // column of a DN one; offsets count codes); in the tile along a row, or down a column where columns are the
        // tile's lines.  Same direction on both sides: bytes move.  Otherwise a thread builds each tile byte from the
        // two codes it holds.
        static_assert(GlobalData::layout == Layout::ND || GlobalData::layout == Layout::DN, "packed fp4 tiles load from ND or DN tensors");
        const auto* g8 = reinterpret_cast<const uint8_t*>(g);
        constexpr bool down = TileData::PairsDownColumns;
        if constexpr (down == (GlobalData::layout == Layout::DN)) {
            for (int idx = threadIdx.x; idx < vr * vc / 2; idx += PTO_AMD_THREADS) {
                int r, c;
                if constexpr (down)
                    c = idx / (vr / 2), r = 2 * (idx - c * (vr / 2));
                else
                    r = idx / (vc / 2), c = 2 * (idx - r * (vc / 2));
                base[dst.ByteOffset(r, c)] = g8[src.Offset(r, c) / 2];
            }
        } else {
            auto code = [&](int r, int c) -> uint32_t {
                const int64_t off = src.Offset(r, c);
                return (g8[off >> 1] >> (4 * (int)(off & 1))) & 0xFu;
            };
            for (int idx = threadIdx.x; idx < vr * vc / 2; idx += PTO_AMD_THREADS) {
                int r, c;
                uint32_t lo, hi;
                if constexpr (down) {
                    r = 2 * (idx / vc), c = idx - (r / 2) * vc;
                    lo = code(r, c), hi = code(r + 1, c);
                } else {
                    c = 2 * (idx / vr), r = idx - (c / 2) * vr;
                    lo = code(r, c), hi = code(r, c + 1);
                }
                base[dst.ByteOffset(r, c)] = (uint8_t)(lo | (hi << 4));
            }
        }
    } else if constexpr (GlobalData::layout == Layout::DN) {  // rows are the contiguous direction in memory
        for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
            const int c = idx / vr, r = idx - c * vr;
            *reinterpret_cast<T*>(base + dst.ByteOffset(r, c)) = g[src.Offset(r, c)];
        }
    } else {
        for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
            const int r = idx / vc, c = idx - r * vc;
            *reinterpret_cast<T*>(base + dst.ByteOffset(r, c)) = g[src.Offset(r, c)];
        }
    }
    __syncthreads();
}

template <typename TileData, typename GlobalData, AtomicType atomic, ReluPreMode relu>
PTO_INST void tstore_lds(GlobalData& dst, TileData& src)
{
    using T = typename TileData::DType;
    using G = typename GlobalData::DType;
    static_assert(atomic == AtomicType::AtomicNone, "TSTORE AtomicAdd from an LDS tile is not implemented on this backend");
    acquire(src);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    auto* g = reinterpret_cast<G*>(dst.data());
    const uint8_t* base = src.Storage();
    if constexpr (is_packed4<T>) {
        static_assert(GlobalData::layout == Layout::ND && sizeof(G) == 1, "packed fp4 tiles store to row-major global tensors");
        for (int idx = threadIdx.x; idx < vr * (vc / 2); idx += PTO_AMD_THREADS) {
            const int r = idx / (vc / 2), c = 2 * (idx - r * (vc / 2));
            if constexpr (TileData::PairsDownColumns) {  // the tile pairs codes down its columns, memory along the row
                const uint32_t lo = (base[src.ByteOffset(r, c)] >> (4 * TileData::Nibble(r, c))) & 0xFu;
                const uint32_t hi = (base[src.ByteOffset(r, c + 1)] >> (4 * TileData::Nibble(r, c + 1))) & 0xFu;
                reinterpret_cast<uint8_t*>(g)[dst.Offset(r, c) / 2] = (uint8_t)(lo | (hi << 4));
            } else {
                reinterpret_cast<uint8_t*>(g)[dst.Offset(r, c) / 2] = base[src.ByteOffset(r, c)];
            }
        }
    } else {
        for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
            const int r = idx / vc, c = idx - r * vc;
            T v = *reinterpret_cast<const T*>(base + src.ByteOffset(r, c));
            if constexpr (is_number<T>) {
                if constexpr (relu == ReluPreMode::NormalRelu)
                    v = v > T(0) ? v : T(0);
                g[dst.Offset(r, c)] = convert<G>(v);
            } else {  // one-byte code types move as bytes
                static_assert(sizeof(G) == sizeof(T), "TSTORE: code tiles store to a global tensor of the same element size");
                reinterpret_cast<T*>(g)[dst.Offset(r, c)] = v;
            }
        }
    }
}

// A Left / Right tile as a window onto the boxed Mat tile it is extracted from: nothing moves, the tile records where
// its lines live.  Possible when the Mat tile stores the lines the matrix unit wants (rows for Left, columns for Right),
// the offset along a line is a whole number of 16-byte chunks, and the window lies inside the source's valid region with
// the destination fully valid (a copy would zero-fill what lies outside; a window cannot).  Returns false when the
// extraction has to copy.
template <typename DstTile, typename SrcTile>
PTO_INST bool textract_window(DstTile& dst, SrcTile& src, int row0, int col0)
{
    using T = typename DstTile::DType;
    if constexpr (SrcTile::MatLines && DstTile::OperandLoc && DstTile::LinesAreRows == SrcTile::LinesAreRows) {
        constexpr bool left = DstTile::LinesAreRows;
        // (fragments are read as 16-byte chunks; the bytes of a scale tile are read one by one, from any offset)
        constexpr bool scale = DstTile::Loc == TileType::ScaleLeft || DstTile::Loc == TileType::ScaleRight;
        const uint32_t kb0 = (uint32_t)(left ? col0 : row0) * (uint32_t)ElemTraits<T>::bytes2 / 2u;  // (packed fp4: two codes per byte)
        const bool ok = (scale || (kb0 & 15u) == 0) && row0 >= 0 && col0 >= 0 && row0 + DstTile::Rows <= src.GetValidRow() &&
                        col0 + DstTile::Cols <= src.GetValidCol() && dst.GetValidRow() == DstTile::Rows &&
                        dst.GetValidCol() == DstTile::Cols;
        if (!ok)
            return false;
        acquire(src);
        dst.lds_ = src.lds_;
        dst.pitch_ = SrcTile::LineBytes;
        dst.sh_ = SrcTile::Swz::sh;
        dst.mask_ = SrcTile::Swz::mask;
        dst.line0_ = (uint32_t)(left ? row0 : col0);
        dst.kb0_ = kb0;
        return true;
    } else {
        return false;
    }
}

// dst(r, c) = src(r + row0, c + col0) over dst's static extent, zero outside src's valid region: the zero fill is what
// lets TMATMUL walk the padded K of Left / Right tiles
// (WINDOW_OK: the caller does not go on to modify the destination, as the relu forms do)
template <bool WINDOW_OK = true, typename DstTile, typename SrcTile>
PTO_INST void textract_lds(DstTile& dst, SrcTile& src, int row0, int col0)
{
    using T = typename DstTile::DType;
    static_assert(std::is_same_v<T, typename SrcTile::DType>, "TMOV / TEXTRACT: element types differ");
    if constexpr (DstTile::OperandLoc) {
        if constexpr (WINDOW_OK) {
            if (textract_window(dst, src, row0, col0))
                return;
        }
        dst.BindOwnLines();  // a copy goes to the tile's own bytes in L0A / L0B
        if (!dst.own_ok_) {
            report(1);  // the TASSIGN address (plus the tile's size) lies outside the region: nothing is copied
            return;
        }
    }
    acquire(src);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const uint8_t* s = src.Storage();
    uint8_t* d = dst.Storage();
    __syncthreads();
    // Transposing move of a whole window: the source keeps the other direction contiguous (a row-major B panel on its way
    // to a Right tile, a column-major A panel to a Left tile).  One thread gathers the 16 / sizeof(T) elements of a
    // destination chunk from consecutive source lines -- neighbouring lanes read neighbouring elements of one line -- and
    // writes the chunk with one 16-byte store.
    if constexpr ((DstTile::Loc == TileType::Left || DstTile::Loc == TileType::Right) && SrcTile::MatLines && !is_packed4<T> &&
                  (sizeof(T) == 1 || sizeof(T) == 2) && DstTile::LinesAreRows != SrcTile::LinesAreRows && DstTile::LineBytes % 16 == 0) {
        if (row0 >= 0 && col0 >= 0 && row0 + DstTile::Rows <= vr && col0 + DstTile::Cols <= vc && dst.GetValidRow() == DstTile::Rows &&
            dst.GetValidCol() == DstTile::Cols) {
            constexpr int EPC = 16 / (int)sizeof(T), chunks = DstTile::LineBytes / 16, units = DstTile::Lines * chunks;
            for (int u = threadIdx.x; u < units; u += PTO_AMD_THREADS) {
                const int line = u % DstTile::Lines, kc = u / DstTile::Lines;
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int e = 0; e < EPC; ++e) {
                    const int kk = kc * EPC + e;
                    const int r = DstTile::LinesAreRows ? line : kk, c = DstTile::LinesAreRows ? kk : line;
                    const uint8_t* sp = s + src.ByteOffset(r + row0, c + col0);
                    const uint32_t v = sizeof(T) == 2 ? (uint32_t)*reinterpret_cast<const uint16_t*>(sp) : (uint32_t)*sp;
                    w[e * (int)sizeof(T) / 4] |= v << (8 * ((e * (int)sizeof(T)) % 4));
                }
                const int r0 = DstTile::LinesAreRows ? line : kc * EPC, c0 = DstTile::LinesAreRows ? kc * EPC : line;
                *reinterpret_cast<uint4*>(d + dst.ByteOffset(r0, c0)) = make_uint4(w[0], w[1], w[2], w[3]);
            }
            __syncthreads();
            return;
        }
    }
    if constexpr (is_packed4<T>) {
        // two fp4 codes per byte: one thread builds one destination byte from the two source nibbles it needs (the
        // pairing direction of source and destination may differ: a Right tile pairs along k, a Mat tile along a row)
        auto code = [&](int r, int c) -> uint32_t {
            const int sr = r + row0, sc = c + col0;
            if (sr < vr && sc < vc && r < dst.GetValidRow() && c < dst.GetValidCol())
                return (s[src.ByteOffset(sr, sc)] >> (4 * SrcTile::Nibble(sr, sc))) & 0xFu;
            return 0u;
        };
        constexpr bool along_rows = DstTile::PairsDownColumns;
        static_assert(along_rows ? DstTile::Rows % 2 == 0 : DstTile::Cols % 2 == 0, "packed fp4 tiles hold element pairs");
        for (int idx = threadIdx.x; idx < DstTile::Rows * DstTile::Cols / 2; idx += PTO_AMD_THREADS) {
            int r, c;
            uint32_t lo, hi;
            if constexpr (along_rows) {
                c = idx / (DstTile::Rows / 2), r = 2 * (idx - c * (DstTile::Rows / 2));
                lo = code(r, c), hi = code(r + 1, c);
            } else {
                r = idx / (DstTile::Cols / 2), c = 2 * (idx - r * (DstTile::Cols / 2));
                lo = code(r, c), hi = code(r, c + 1);
            }
            d[dst.ByteOffset(r, c)] = (uint8_t)(lo | (hi << 4));
        }
    } else if constexpr (DstTile::Loc == TileType::Right) {  // stored transposed: walk k (rows) fastest
        for (int idx = threadIdx.x; idx < DstTile::Rows * DstTile::Cols; idx += PTO_AMD_THREADS) {
            const int c = idx / DstTile::Rows, r = idx - c * DstTile::Rows;
            const int sr = r + row0, sc = c + col0;
            T v{};
            if (sr < vr && sc < vc && r < dst.GetValidRow() && c < dst.GetValidCol())
                v = *reinterpret_cast<const T*>(s + src.ByteOffset(sr, sc));
            *reinterpret_cast<T*>(d + dst.ByteOffset(r, c)) = v;
        }
    } else {
        for (int idx = threadIdx.x; idx < DstTile::Rows * DstTile::Cols; idx += PTO_AMD_THREADS) {
            const int r = idx / DstTile::Cols, c = idx - r * DstTile::Cols;
            const int sr = r + row0, sc = c + col0;
            T v{};
            if (sr < vr && sc < vc && r < dst.GetValidRow() && c < dst.GetValidCol())
                v = *reinterpret_cast<const T*>(s + src.ByteOffset(sr, sc));
            *reinterpret_cast<T*>(d + dst.ByteOffset(r, c)) = v;
        }
    }
    __syncthreads();
}

// ---- the contraction ------------------------------------------------------------------------------------------------
// One 32 x 32 block per MFMA chain.  Lane (l32, lhi) feeds line l32 of an operand block (a row of Left, a column of
// Right); its k-slots inside a step are lhi * (STEP / 2) .. + STEP / 2 - 1, read as one fragment of 4, 8 or 16 bytes.
// The Right fragment goes in as the instruction's first operand, so the result block arrives transposed: the lane holds
// row l32 of C and four consecutive columns per register quad.
template <typename T>
struct Mfma;
template <>
struct Mfma<_Float16> {
    static constexpr int STEP = 16;
    using Frag = f16x8;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c, 0, 0, 0); }
};
template <>
struct Mfma<__bf16> {
    static constexpr int STEP = 16;
    using Frag = bf16x8;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c, 0, 0, 0); }
};
template <>
struct Mfma<int8_t> {
    static constexpr int STEP = 32;
    using Frag = i32x4v;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, c, 0, 0, 0); }
};
template <>
struct Mfma<float> {
    static constexpr int STEP = 2;
    using Frag = float;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, c, 0, 0, 0); }
};
template <>
struct Mfma<float8_e4m3_t> {
    static constexpr int STEP = 16;
    using Frag = long;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b, a, c, 0, 0, 0); }
};
template <>
struct Mfma<float8_e5m2_t> {
    static constexpr int STEP = 16;
    using Frag = long;
    template <typename Acc>
    PTO_INST static Acc run(Frag a, Frag b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(b, a, c, 0, 0, 0); }
};

// compile-time loop with literal indices (register arrays stay in registers)
template <int... Is, class F>
PTO_INST void static_for_impl(std::integer_sequence<int, Is...>, F&& f)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
PTO_INST void static_for(F&& f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

template <bool INIT, typename TileRes, typename TileLeftT, typename TileRightT>
PTO_INST void tmatmul(TileRes& c, TileLeftT& a, TileRightT& b)
{
    using T = typename TileLeftT::DType;
    static_assert(TileRes::Loc == TileType::Acc && TileLeftT::Loc == TileType::Left && TileRightT::Loc == TileType::Right,
                  "TMATMUL takes (Acc, Left, Right) tiles");
    static_assert(std::is_same_v<T, typename TileRightT::DType>, "TMATMUL: Left and Right element types differ");
    static_assert(TileLeftT::Cols == TileRightT::Rows && TileRes::Rows == TileLeftT::Rows && TileRes::Cols == TileRightT::Cols,
                  "TMATMUL: static tile shapes do not chain (M x K) . (K x N) -> (M x N)");
    static_assert(std::is_integral_v<typename TileRes::DType> == std::is_integral_v<T>,
                  "TMATMUL: int8 operands accumulate in int32, floating operands in float");
    using M = Mfma<T>;
    using Frag = typename M::Frag;
    static_assert(TileLeftT::Cols % M::STEP == 0, "TMATMUL: the static K of the tiles must be a multiple of the MFMA k-step");
    const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint8_t* pa = a.Storage();
    const uint8_t* pb = b.Storage();
    if constexpr (INIT) {
#pragma unroll
        for (int slot = 0; slot < TileRes::NBLK; ++slot)
            c.regs[slot] = typename TileRes::Vec16(0);
    }
    if constexpr (TileRes::BLOCKED) {
        // The wave owns MB x NB neighbouring blocks: per k-step it reads MB Left and NB Right fragments and issues
        // MB * NB MFMAs.  A lane's line is the same in every k-step, so the line part of the address is computed once.
        constexpr int MB = TileRes::MB, NB = TileRes::NB;
        const int wr = wave / TileRes::grid.wc, wc = wave % TileRes::grid.wc;
        uint32_t aline[MB], bline[NB];
#pragma unroll
        for (int i = 0; i < MB; ++i)
            aline[i] = (uint32_t)min((wr * MB + i) * 32 + l32, TileLeftT::Rows - 1);
#pragma unroll
        for (int j = 0; j < NB; ++j)
            bline[j] = (uint32_t)min((wc * NB + j) * 32 + l32, TileRightT::Cols - 1);
        auto kstep = [&](int k0) __attribute__((always_inline)) {
            const int k = k0 + lhi * (M::STEP / 2);
            Frag fa[MB], fb[NB];
#pragma unroll
            for (int j = 0; j < NB; ++j)
                fb[j] = *reinterpret_cast<const Frag*>(pb + b.ByteOffset(k, (int)bline[j]));
#pragma unroll
            for (int i = 0; i < MB; ++i)
                fa[i] = *reinterpret_cast<const Frag*>(pa + a.ByteOffset((int)aline[i], k));
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    c.regs[i * NB + j] = M::run(fa[i], fb[j], c.regs[i * NB + j]);
        };
        if constexpr (TileLeftT::ValidCol != DYNAMIC) {  // the padded K is known: a straight line of k-steps
            constexpr int kpad = (TileLeftT::ValidCol + M::STEP - 1) / M::STEP * M::STEP < TileLeftT::Cols
                                     ? (TileLeftT::ValidCol + M::STEP - 1) / M::STEP * M::STEP
                                     : TileLeftT::Cols;
            static_for<kpad / M::STEP>([&](auto sc) { kstep(decltype(sc)::value * M::STEP); });
        } else {
            const int kpad = min((a.GetValidCol() + M::STEP - 1) / M::STEP * M::STEP, TileLeftT::Cols);
            for (int k0 = 0; k0 < kpad; k0 += M::STEP)
                kstep(k0);
        }
    } else {
        const int kpad = min((a.GetValidCol() + M::STEP - 1) / M::STEP * M::STEP, TileLeftT::Cols);
#pragma unroll
        for (int slot = 0; slot < TileRes::NBLK; ++slot) {
            int bi, bj;
            if (TileRes::block_of(slot, wave, bi, bj)) {
                const int arow = min(bi * 32 + l32, TileLeftT::Rows - 1);
                const int bcol = min(bj * 32 + l32, TileRightT::Cols - 1);
                typename TileRes::Vec16 acc = c.regs[slot];
                for (int k0 = 0; k0 < kpad; k0 += M::STEP) {
                    const int k = k0 + lhi * (M::STEP / 2);
                    acc = M::run(*reinterpret_cast<const Frag*>(pa + a.ByteOffset(arow, k)),
                                 *reinterpret_cast<const Frag*>(pb + b.ByteOffset(k, bcol)), acc);
                }
                c.regs[slot] = acc;
            }
        }
    }
}

// Block-scaled contraction on v_mfma_scale_f32_32x32x64_f8f6f4: a k-step is two MX blocks of 32; lane (l32, lhi) feeds
// bytes [16 lhi, 16 lhi + 16) of each block of its row / column and the E8M0 scale of block lhi.  As in tmatmul the Right
// operand (with its scale) goes first, so the accumulator block arrives transposed.
template <typename T>
struct MxFormat;
template <>
struct MxFormat<float8_e4m3_t> {
    static constexpr int code = 0;
};
template <>
struct MxFormat<float8_e5m2_t> {
    static constexpr int code = 1;
};
template <>
struct MxFormat<float4_e2m1x2_t> {
    static constexpr int code = 4;
};
template <>
struct MxFormat<float4_e1m2x2_t> {
    static constexpr int code = 0;  // the scaled MFMA has no E1M2 format: such operands are widened to E4M3 first
};
typedef int i32x8v __attribute__((ext_vector_type(8)));

// Packed fp4 codes -> E4M3 bytes, exactly: every E2M1 value (0 .. 6) and every E1M2 value (0 .. 1.75) is an E4M3 number.
// The scaled MFMA has no E1M2 format, so E1M2 operands (and an E2M1 operand paired with one) run as fp8.
template <typename T>
PTO_INST uint2 fp4x8_to_e4m3(uint32_t packed)
{
    // E4M3 codes of the eight magnitudes, one byte each, low magnitude in the low byte
    constexpr uint32_t lo = std::is_same_v<T, float4_e1m2x2_t> ? 0x34302800u : 0x3C383000u;   // E1M2: 0, .25, .5, .75 | E2M1: 0, .5, 1, 1.5
    constexpr uint32_t hi = std::is_same_v<T, float4_e1m2x2_t> ? 0x3E3C3A38u : 0x4C484440u;   // E1M2: 1, 1.25, 1.5, 1.75 | E2M1: 2, 3, 4, 6
    uint2 out;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const uint32_t x = (packed >> (16 * half)) & 0xFFFFu;   // four codes
        const uint32_t spread = (x & 0xFu) | ((x & 0xF0u) << 4) | ((x & 0xF00u) << 8) | ((x & 0xF000u) << 12);   // one code per byte
        const uint32_t mag = __builtin_amdgcn_perm(hi, lo, spread & 0x07070707u);   // byte i of the result = table[code i & 7]
        const uint32_t v = mag | ((spread & 0x08080808u) << 4);
        if (half == 0)
            out.x = v;
        else
            out.y = v;
    }
    return out;
}

template <bool INIT, typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT>
PTO_INST void tmatmul_mx(TileRes& c, TileLeftT& a, TileLeftScaleT& as, TileRightT& b, TileRightScaleT& bs)
{
    using TA = typename TileLeftT::DType;
    using TB = typename TileRightT::DType;
    static_assert(TileRes::Loc == TileType::Acc && TileLeftT::Loc == TileType::Left && TileRightT::Loc == TileType::Right &&
                      TileLeftScaleT::Loc == TileType::ScaleLeft && TileRightScaleT::Loc == TileType::ScaleRight,
                  "TMATMUL_MX takes (Acc, Left, ScaleLeft, Right, ScaleRight) tiles");
    static_assert(std::is_same_v<typename TileRes::DType, float>, "TMATMUL_MX accumulates in float");
    static_assert(is_packed4<TA> == is_packed4<TB>, "TMATMUL_MX: both operands fp8 or both fp4");
    static_assert(TileLeftT::Cols % 64 == 0, "TMATMUL_MX: the static K of the Left tile must be a multiple of 64");
    // a one-row Left tile (TGEMV_MX) may be declared wider than the Right tile is tall, and meets a 16-row accumulator
    constexpr bool gemv = TileLeftT::Rows == 1;
    static_assert((TileLeftT::Cols == TileRightT::Rows || (gemv && TileLeftT::Cols >= TileRightT::Rows)) &&
                      (TileRes::Rows == TileLeftT::Rows || gemv) && TileRes::Cols == TileRightT::Cols,
                  "TMATMUL_MX: static tile shapes do not chain");
    // (scale tiles may be declared larger than the K / 32 groups they hold)
    static_assert(TileLeftScaleT::Rows == TileLeftT::Rows && TileLeftScaleT::Cols * 32 >= TileRightT::Rows &&
                      TileRightScaleT::Cols == TileRightT::Cols && TileRightScaleT::Rows * 32 >= TileRightT::Rows,
                  "TMATMUL_MX: one E8M0 scale per 32 K-elements");
    constexpr bool via_fp8 = std::is_same_v<TA, float4_e1m2x2_t> || std::is_same_v<TB, float4_e1m2x2_t>;
    const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kpad = min((a.GetValidCol() + 63) / 64 * 64, TileRightT::Rows);
    const uint8_t *pa = a.Storage(), *pb = b.Storage(), *psa = as.Storage(), *psb = bs.Storage();
    if constexpr (TileRes::BLOCKED && !via_fp8 && !gemv) {
        // fp8 / fp4 on a wave grid: per k-step (two MX blocks) the wave reads the fragments and scale bytes of its MB row
        // blocks and NB column blocks once and issues MB * NB scaled MFMAs (as tmatmul does for the plain types).  A k-step
        // is 64 bytes of a line of fp8 codes -- a lane holds 16 bytes of either block -- and 32 bytes of packed fp4 codes --
        // a lane holds the 16 bytes that are block lhi.
        constexpr int MB = TileRes::MB, NB = TileRes::NB;
        const int wr = wave / TileRes::grid.wc, wc = wave % TileRes::grid.wc;
        int aline[MB], bline[NB];
#pragma unroll
        for (int i = 0; i < MB; ++i)
            aline[i] = min((wr * MB + i) * 32 + l32, TileLeftT::Rows - 1);
#pragma unroll
        for (int j = 0; j < NB; ++j)
            bline[j] = min((wc * NB + j) * 32 + l32, TileRightT::Cols - 1);
        if constexpr (INIT) {
#pragma unroll
            for (int slot = 0; slot < TileRes::NBLK; ++slot)
                c.regs[slot] = typename TileRes::Vec16(0);
        }
        // Fragment addresses.  A lane reads line l32 of every block of its wave tile; blocks are 32 lines apart, which
        // leaves the swizzle term (line >> sh) & mask unchanged, so the chunk at 16-byte index c of block i lies at
        //     line0 * pitch + ((c ^ swz) << 4) + i * 32 * pitch.
        // With c = c0 + lhi and c0 even, (c0 + lhi) ^ swz = c0 ^ (lhi ^ swz): one lane constant per operand XOR a literal,
        // plus a literal block offset that goes into the read instruction.  Written out here because, computed block by
        // block through ByteOffset, every address is its own loop-invariant value, and a program's worth of them does not
        // fit the register file next to the accumulators.  (Needs a power-of-two number of chunks per line and windows
        // that start on 32-byte boundaries along K; anything else takes ByteOffset.)
        const uint8_t* arena = lds_arena();
        const uint32_t a_l0 = (uint32_t)(wr * MB * 32 + l32) + a.line0_, b_l0 = (uint32_t)(wc * NB * 32 + l32) + b.line0_;
        const bool fast_addr = (a.pitch_ & (a.pitch_ - 1)) == 0 && (b.pitch_ & (b.pitch_ - 1)) == 0 && a.pitch_ >= 64 && b.pitch_ >= 64 &&
                               (a.kb0_ & 31u) == 0 && (b.kb0_ & 31u) == 0;
        const uint32_t a_lane = a.lds_ + a_l0 * a.pitch_ + (((uint32_t)lhi ^ ((a_l0 >> a.sh_) & a.mask_)) << 4);
        const uint32_t b_lane = b.lds_ + b_l0 * b.pitch_ + (((uint32_t)lhi ^ ((b_l0 >> b.sh_) & b.mask_)) << 4);
        constexpr bool fp4 = is_packed4<TA>;
        auto frag = [&](bool left, int blk, int kbyte) __attribute__((always_inline)) -> uint4 {
            // kbyte: the k-step's first byte along the line, or 32 past it (fp8): a literal multiple of 32
            if (fast_addr) {
                const uint32_t lane_c = left ? a_lane : b_lane, pitch = left ? a.pitch_ : b.pitch_, kb0 = left ? a.kb0_ : b.kb0_;
                return *reinterpret_cast<const uint4*>(arena + ((lane_c ^ (kb0 + (uint32_t)kbyte)) + (uint32_t)blk * 32u * pitch));
            }
            const int k_el = fp4 ? 2 * (kbyte + 16 * lhi) : kbyte + 16 * lhi;  // ByteOffset takes element indices
            return left ? *reinterpret_cast<const uint4*>(pa + a.ByteOffset(aline[blk], k_el))
                        : *reinterpret_cast<const uint4*>(pb + b.ByteOffset(k_el, bline[blk]));
        };
        auto kstep = [&](int k0) __attribute__((always_inline)) {
            const int g = k0 / 32 + lhi;
            i32x8v fa[MB], fb[NB];
            int sa[MB], sb[NB];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                if constexpr (fp4) {
                    const uint4 b0 = frag(false, j, k0 / 2);
                    fb[j] = i32x8v{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, 0, 0, 0, 0};
                } else {
                    const uint4 b0 = frag(false, j, k0), b1 = frag(false, j, k0 + 32);
                    fb[j] = i32x8v{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
                }
                sb[j] = psb[bs.ByteOffset(g, bline[j])];
            }
#pragma unroll
            for (int i = 0; i < MB; ++i) {
                if constexpr (fp4) {
                    const uint4 a0 = frag(true, i, k0 / 2);
                    fa[i] = i32x8v{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, 0, 0, 0, 0};
                } else {
                    const uint4 a0 = frag(true, i, k0), a1 = frag(true, i, k0 + 32);
                    fa[i] = i32x8v{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                }
                sa[i] = psa[as.ByteOffset(aline[i], g)];
            }
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    c.regs[i * NB + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], c.regs[i * NB + j], MxFormat<TB>::code,
                                                                                         MxFormat<TA>::code, 0, sb[j], 0, sa[i]);
        };
        if constexpr (TileLeftT::ValidCol != DYNAMIC) {
            constexpr int kp = (TileLeftT::ValidCol + 63) / 64 * 64 < TileRightT::Rows ? (TileLeftT::ValidCol + 63) / 64 * 64 : TileRightT::Rows;
            static_for<kp / 64>([&](auto sc) { kstep(decltype(sc)::value * 64); });
        } else {
            for (int k0 = 0; k0 < kpad; k0 += 64)
                kstep(k0);
        }
        // The MFMAs are register-to-register operations that the compiler may move freely, and it sinks them past the
        // next instructions' barriers and branches to where the accumulators are next needed -- with every fragment
        // they read kept live until then.  An empty statement that "uses" the accumulators pins them to this call.
#pragma unroll
        for (int slot = 0; slot < TileRes::NBLK; ++slot)
            asm volatile("" : "+v"(c.regs[slot]));
        return;
    }
#pragma unroll
    for (int slot = 0; slot < TileRes::NBLK; ++slot) {
        int bi, bj;
        if (TileRes::block_of(slot, wave, bi, bj)) {
            const int arow = min(bi * 32 + l32, TileLeftT::Rows - 1);
            const int bcol = min(bj * 32 + l32, TileRightT::Cols - 1);
            typename TileRes::Vec16 acc = c.regs[slot];
            if constexpr (INIT)
                acc = typename TileRes::Vec16(0);
            for (int k0 = 0; k0 < kpad; k0 += 64) {
                const int g = k0 / 32 + lhi;
                const int sa = psa[as.ByteOffset(arow, g)], sb = psb[bs.ByteOffset(g, bcol)];
                i32x8v av = {0, 0, 0, 0, 0, 0, 0, 0}, bv = {0, 0, 0, 0, 0, 0, 0, 0};
                if constexpr (via_fp8) {  // fp4 codes widened to E4M3 bytes, then fed like fp8: 16 elements of each block per lane
                    const uint2 a0 = *reinterpret_cast<const uint2*>(pa + a.ByteOffset(arow, k0 + 16 * lhi));
                    const uint2 a1 = *reinterpret_cast<const uint2*>(pa + a.ByteOffset(arow, k0 + 32 + 16 * lhi));
                    const uint2 b0 = *reinterpret_cast<const uint2*>(pb + b.ByteOffset(k0 + 16 * lhi, bcol));
                    const uint2 b1 = *reinterpret_cast<const uint2*>(pb + b.ByteOffset(k0 + 32 + 16 * lhi, bcol));
                    const uint2 ea[4] = {fp4x8_to_e4m3<TA>(a0.x), fp4x8_to_e4m3<TA>(a0.y), fp4x8_to_e4m3<TA>(a1.x), fp4x8_to_e4m3<TA>(a1.y)};
                    const uint2 eb[4] = {fp4x8_to_e4m3<TB>(b0.x), fp4x8_to_e4m3<TB>(b0.y), fp4x8_to_e4m3<TB>(b1.x), fp4x8_to_e4m3<TB>(b1.y)};
                    av = i32x8v{(int)ea[0].x, (int)ea[0].y, (int)ea[1].x, (int)ea[1].y, (int)ea[2].x, (int)ea[2].y, (int)ea[3].x, (int)ea[3].y};
                    bv = i32x8v{(int)eb[0].x, (int)eb[0].y, (int)eb[1].x, (int)eb[1].y, (int)eb[2].x, (int)eb[2].y, (int)eb[3].x, (int)eb[3].y};
                    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, acc, 0, 0, 0, sb, 0, sa);
                } else {
                    if constexpr (is_packed4<TA>) {  // fp4: the lane's 16 bytes are the whole MX block lhi
                        const uint4 a0 = *reinterpret_cast<const uint4*>(pa + a.ByteOffset(arow, k0 + 32 * lhi));
                        const uint4 b0 = *reinterpret_cast<const uint4*>(pb + b.ByteOffset(k0 + 32 * lhi, bcol));
                        av = i32x8v{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, 0, 0, 0, 0};
                        bv = i32x8v{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, 0, 0, 0, 0};
                    } else {  // fp8: bytes [16 lhi, 16 lhi + 16) of each of the two blocks
                        const uint4 a0 = *reinterpret_cast<const uint4*>(pa + a.ByteOffset(arow, k0 + 16 * lhi));
                        const uint4 a1 = *reinterpret_cast<const uint4*>(pa + a.ByteOffset(arow, k0 + 32 + 16 * lhi));
                        const uint4 b0 = *reinterpret_cast<const uint4*>(pb + b.ByteOffset(k0 + 16 * lhi, bcol));
                        const uint4 b1 = *reinterpret_cast<const uint4*>(pb + b.ByteOffset(k0 + 32 + 16 * lhi, bcol));
                        av = i32x8v{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                        bv = i32x8v{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
                    }
                    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, acc, MxFormat<TB>::code, MxFormat<TA>::code, 0, sb, 0, sa);
                }
            }
            c.regs[slot] = acc;
        }
    }
}

// visits every accumulator element this lane owns: f(slot, reg index, row, col)
template <typename TileRes, typename F>
PTO_INST void for_each_acc(TileRes& c, F&& f)
{
    const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int slot = 0; slot < TileRes::NBLK; ++slot) {
        int bi, bj;
        if (TileRes::block_of(slot, wave, bi, bj)) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                f(slot, r, bi * 32 + l32, bj * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3));
        }
    }
}

template <typename G>
struct alignas(4 * sizeof(G)) Quad {
    G v[4];
};

template <typename G>
PTO_INST void stage_quad(uint8_t* at, const Quad<G>& q)
{
    if constexpr (sizeof(G) == 2)
        *reinterpret_cast<i32x2s*>(at) = __builtin_bit_cast(i32x2v_plain, q);
    else
        *reinterpret_cast<i32x4s*>(at) = __builtin_bit_cast(i32x4v, q);
}

template <typename TileRes, typename GlobalData, AtomicType atomic, ReluPreMode relu>
PTO_INST void tstore_acc(GlobalData& dst, TileRes& src)
{
    using G = typename GlobalData::DType;
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    auto* g = reinterpret_cast<G*>(dst.data());
    // Row-major destination with unit column stride: a lane's register quad is four consecutive columns of one row, so
    // it leaves as one 8- or 16-byte store where the quad is whole and aligned.
    if constexpr (GlobalData::layout == Layout::ND && atomic == AtomicType::AtomicNone && (sizeof(G) == 2 || sizeof(G) == 4)) {
        const int64_t ld = dst.GetStride(3);
        const bool vec_ok = dst.GetShape(0) == 1 && dst.GetShape(1) == 1 && dst.GetShape(2) == 1 && dst.GetStride(4) == 1 &&
                            (ld & 3) == 0 && (reinterpret_cast<uintptr_t>(g) & (4 * sizeof(G) - 1)) == 0 && vr <= dst.GetShape(3);
        if (vec_ok) {
            const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
            const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            // Whole tile, whole blocks, 16-byte aligned rows, and a staging band per wave: every block goes through LDS
            // and leaves as whole rows (64 or 128 contiguous bytes per row and store instruction).  The band is private
            // to the wave, so no workgroup barrier is involved.
            constexpr int row_bytes = 32 * (int)sizeof(G), pitch = row_bytes + 16, band = 32 * pitch;
            // 16-bit outputs, two blocks side by side in one wave: the pair is staged 16 rows at a time, so that a row
            // leaves as 128 contiguous bytes (a whole cache line per row, where 64-byte halves from two instructions
            // cost extra write traffic).  Same band size or less: 16 rows of 128 + 16 bytes.
            constexpr bool pair = sizeof(G) == 2 && TileRes::BLOCKED && TileRes::NB % 2 == 0;
            constexpr int pair_pitch = 128 + 16, pair_band = 16 * pair_pitch;
            if constexpr (pair && TileRes::Rows % 32 == 0 && TileRes::Cols % 32 == 0 &&
                          (uint32_t)(WAVES * pair_band) <= (uint32_t)PTO_AMD_STAGE_BYTES) {
                if (vr == TileRes::Rows && vc == TileRes::Cols && ((ld * (int64_t)sizeof(G)) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
                    if constexpr (STAGE_ALIASES_L1)
                        __syncthreads();  // every wave has read its last operands out of L1
                    uint8_t* stage = lds_arena() + STAGE_BASE + wave * pair_band;
#pragma unroll
                    for (int slot = 0; slot < TileRes::NBLK; slot += 2) {
                        int bi, bj;
                        TileRes::block_of(slot, wave, bi, bj);
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
                            if ((l32 >> 4) == half) {
#pragma unroll
                                for (int blk = 0; blk < 2; ++blk) {
#pragma unroll
                                    for (int q = 0; q < 4; ++q) {
                                        Quad<G> out;
#pragma unroll
                                        for (int e = 0; e < 4; ++e) {
                                            auto v = src.regs[slot + blk][4 * q + e];
                                            if constexpr (relu == ReluPreMode::NormalRelu)
                                                v = v > 0 ? v : 0;
                                            out.v[e] = convert<G>(v);
                                        }
                                        stage_quad(stage + (l32 & 15) * pair_pitch + blk * 64 + (8 * q + 4 * lhi) * 2, out);
                                    }
                                }
                            }
                            __builtin_amdgcn_wave_barrier();
#pragma unroll
                            for (int pass = 0; pass < 2; ++pass) {
                                const int idx = lane + 64 * pass, r = idx >> 3, chunk = idx & 7;
                                const i32x4v v = *reinterpret_cast<const i32x4s*>(stage + r * pair_pitch + chunk * 16);
                                uint8_t* gp = reinterpret_cast<uint8_t*>(g + (int64_t)(bi * 32 + half * 16 + r) * ld + bj * 32) + chunk * 16;
                                __builtin_nontemporal_store(v, reinterpret_cast<i32x4v*>(gp));
                            }
                            __builtin_amdgcn_wave_barrier();
                        }
                    }
                    return;
                }
            }
            if constexpr (TileRes::Rows % 32 == 0 && TileRes::Cols % 32 == 0 && (uint32_t)(WAVES * band) <= (uint32_t)PTO_AMD_STAGE_BYTES) {
                if (vr == TileRes::Rows && vc == TileRes::Cols && ((ld * (int64_t)sizeof(G)) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
                    if constexpr (STAGE_ALIASES_L1)
                        __syncthreads();
                    uint8_t* stage = lds_arena() + STAGE_BASE + wave * band;
                    constexpr int lanes_per_row = row_bytes / 16, rows_per_pass = 64 / lanes_per_row;
                    const int rrow = lane / lanes_per_row, rchunk = lane % lanes_per_row;
#pragma unroll
                    for (int slot = 0; slot < TileRes::NBLK; ++slot) {
                        int bi, bj;
                        TileRes::block_of(slot, wave, bi, bj);
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            Quad<G> out;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                auto v = src.regs[slot][4 * q + e];
                                if constexpr (relu == ReluPreMode::NormalRelu)
                                    v = v > 0 ? v : 0;
                                out.v[e] = convert<G>(v);
                            }
                            stage_quad(stage + l32 * pitch + (8 * q + 4 * lhi) * (int)sizeof(G), out);
                        }
                        __builtin_amdgcn_wave_barrier();
#pragma unroll
                        for (int pass = 0; pass < 32 / rows_per_pass; ++pass) {
                            const int r = pass * rows_per_pass + rrow;
                            const i32x4v v = *reinterpret_cast<const i32x4s*>(stage + r * pitch + rchunk * 16);
                            uint8_t* gp = reinterpret_cast<uint8_t*>(g + (int64_t)(bi * 32 + r) * ld + bj * 32) + rchunk * 16;
                            __builtin_nontemporal_store(v, reinterpret_cast<i32x4v*>(gp));
                        }
                        __builtin_amdgcn_wave_barrier();
                    }
                    return;
                }
            }
#pragma unroll
            for (int slot = 0; slot < TileRes::NBLK; ++slot) {
                int bi, bj;
                if (TileRes::block_of(slot, wave, bi, bj)) {
                    const int row = bi * 32 + l32;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int col = bj * 32 + 8 * q + 4 * lhi;
                        if (row < vr && col + 3 < vc) {
                            Quad<G> out;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                auto v = src.regs[slot][4 * q + e];
                                if constexpr (relu == ReluPreMode::NormalRelu)
                                    v = v > 0 ? v : 0;
                                out.v[e] = convert<G>(v);
                            }
                            *reinterpret_cast<Quad<G>*>(g + (int64_t)row * ld + col) = out;
                        } else if (row < vr) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                if (col + e < vc) {
                                    auto v = src.regs[slot][4 * q + e];
                                    if constexpr (relu == ReluPreMode::NormalRelu)
                                        v = v > 0 ? v : 0;
                                    g[(int64_t)row * ld + col + e] = convert<G>(v);
                                }
                            }
                        }
                    }
                }
            }
            return;
        }
    }
    for_each_acc(src, [&](int slot, int r, int row, int col) {
        if (row < vr && col < vc) {
            auto v = src.regs[slot][r];
            if constexpr (relu == ReluPreMode::NormalRelu)
                v = v > 0 ? v : 0;
            if constexpr (atomic == AtomicType::AtomicAdd) {
                static_assert(atomic != AtomicType::AtomicAdd || std::is_same_v<G, float> || std::is_same_v<G, int32_t>,
                              "TSTORE AtomicAdd targets float or int32 on this backend");
                atomicAdd(&g[dst.Offset(row, col)], convert<G>(v));
            } else {
                g[dst.Offset(row, col)] = convert<G>(v);
            }
        }
    });
}

// Fix-pipe quantisation of one accumulator element (reference: cpu/common.hpp:117-185).  Scalar words carry an fp32
// scale in the low 32 bits; vector (per-column) words a 19-bit (1, 8, 10) float at bits 13..31.  Bits 37..45 hold the
// offset and bit 46 the signedness of 8-bit targets.
template <bool VECTOR>
PTO_INST float quant_word_scale(uint64_t word)
{
    return ptoamd::fixpipe_word_scale<VECTOR>(word);
}
// sat_inf: bit 48 of the task cookie, read once per instruction by the caller
template <bool VECTOR, typename G, typename Reg>
PTO_INST float quantize_element(Reg acc, uint64_t word, bool sat_inf = false)
{
    constexpr bool src_is_int = std::is_integral_v<Reg>;
    static_assert(std::is_same_v<G, int8_t> || std::is_same_v<G, uint8_t> || std::is_same_v<G, _Float16> || std::is_same_v<G, __bf16> ||
                      (std::is_same_v<G, int16_t> && src_is_int),
                  "fix-pipe quantisation targets int8, uint8, half or bfloat16 (and int16 from an int32 accumulator)");
    float r = __fmul_rn((float)acc, quant_word_scale<VECTOR>(word));
    if constexpr (std::is_same_v<G, int16_t>) {
        // shift mode (cpu/common.hpp:174-180): arithmetic shift right by bits 32..35 of the word plus one; the
        // reference narrows to int16 before it clamps, so the value wraps
        const int shift = (int)((word >> 32) & 0xFu) + 1;
        r = (float)(int16_t)((int32_t)acc >> shift);
    } else if constexpr (sizeof(G) == 1) {
        r = ptoamd::fixpipe_quantize<VECTOR, true, src_is_int>((float)acc, word);
    } else if constexpr (std::is_same_v<G, _Float16>) {
        if (!src_is_int && sat_inf)
            r = ptoamd::fixpipe_saturate_inf<true>(r);
        else
            r = ptoamd::fixpipe_quantize<VECTOR, false, src_is_int>((float)acc, word);
    } else {
        if (sat_inf)
            r = ptoamd::fixpipe_saturate_inf<false>(r);
        else if (r == r && fabsf(r) != __builtin_inff())
            r = r < -3.402823466e38f ? -3.402823466e38f : (r > 3.402823466e38f ? 3.402823466e38f : r);
    }
    return r;
}

// The same from an on-chip buffer tile (the reference's TSTORE quantises whatever tile it is given, cpu/TStore.hpp:41-62;
// its tstore_quant tests drain Vec tiles of float / int32): element by element over the valid region.
template <bool VECTOR, typename TileData, typename GlobalData, ReluPreMode relu, typename WordOf>
PTO_INST void tstore_lds_quant(GlobalData& dst, TileData& src, WordOf&& word_of)
{
    using T = typename TileData::DType;
    using G = typename GlobalData::DType;
    static_assert(std::is_same_v<T, float> || std::is_same_v<T, int32_t>, "the fix-pipe quantises float or int32 values");
    acquire(src);
    __syncthreads();  // writers of the tile (and of the Scaling tile the words come from) are done
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    auto* g = reinterpret_cast<G*>(dst.data());
    const uint8_t* base = src.Storage();
    const bool sat_inf = (get_task_cookie() >> 48) & 1u;
    for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
        const int r = idx / vc, c = idx - r * vc;
        float v = quantize_element<VECTOR, G>(*reinterpret_cast<const T*>(base + src.ByteOffset(r, c)), word_of(c), sat_inf);
        if constexpr (relu == ReluPreMode::NormalRelu)
            v = v > 0 ? v : 0;
        g[dst.Offset(r, c)] = static_cast<G>(v);
    }
}

template <bool VECTOR, typename TileRes, typename GlobalData, ReluPreMode relu, typename WordOf>
PTO_INST void tstore_acc_quant(GlobalData& dst, TileRes& src, WordOf&& word_of)
{
    using G = typename GlobalData::DType;
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    auto* g = reinterpret_cast<G*>(dst.data());
    const bool sat_inf = (get_task_cookie() >> 48) & 1u;
    for_each_acc(src, [&](int slot, int r, int row, int col) {
        if (row < vr && col < vc) {
            float v = quantize_element<VECTOR, G>(src.regs[slot][r], word_of(col), sat_inf);
            if constexpr (relu == ReluPreMode::NormalRelu)
                v = v > 0 ? v : 0;
            g[dst.Offset(row, col)] = static_cast<G>(v);
        }
    });
}

}  // namespace amd

// ---- TLOAD ---------------------------------------------------------------------------------------------------------
template <typename TileData, typename GlobalData, typename... WaitEvents>
PTO_INST RecordEvent TLOAD(TileData& dst, GlobalData& src, WaitEvents&...)
{
    static_assert(TileData::Loc != TileType::Acc, "TLOAD targets an on-chip buffer tile, not an accumulator");
    PTO_AMD_TRACE_INSTR(1, TR_TLOAD, dst, src);
    amd::tload_lds(dst, src);
    return {};
}

// ---- TSTORE --------------------------------------------------------------------------------------------------------
template <typename TileData, typename GlobalData, AtomicType atomicType = AtomicType::AtomicNone,
          ReluPreMode reluPreMode = ReluPreMode::NoRelu, typename... WaitEvents>
PTO_INST RecordEvent TSTORE(GlobalData& dst, TileData& src, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TSTORE, dst, src);
    if constexpr (TileData::Loc == TileType::Acc)
        amd::tstore_acc<TileData, GlobalData, atomicType, reluPreMode>(dst, src);
    else
        amd::tstore_lds<TileData, GlobalData, atomicType, reluPreMode>(dst, src);
    return {};
}

// TSTORE with fix-pipe quantisation: one scalar word for the whole tile, or one word per column from a Scaling tile
// (reference: common/pto_instr.hpp:439-490, cpu/TStore.hpp:118-181)
template <typename TileData, typename GlobalData, AtomicType atomicType = AtomicType::AtomicNone,
          ReluPreMode reluPreMode = ReluPreMode::NoRelu>
PTO_INST RecordEvent TSTORE(GlobalData& dst, TileData& src, uint64_t preQuantScalar)
{
    PTO_AMD_TRACE_INSTR(1, TR_TSTORE, dst, src);
    static_assert(atomicType == AtomicType::AtomicNone, "the quantising TSTORE does not add atomically");
    if constexpr (TileData::Loc == TileType::Acc)
        amd::tstore_acc_quant<false, TileData, GlobalData, reluPreMode>(dst, src, [&](int) { return preQuantScalar; });
    else
        amd::tstore_lds_quant<false, TileData, GlobalData, reluPreMode>(dst, src, [&](int) { return preQuantScalar; });
    return {};
}
// (the words come from a Scaling tile, or -- as the reference's tstore_quant tests have it -- from a one-row Vec tile of
// 64-bit elements)
template <typename TileData, typename GlobalData, typename FpTileData, AtomicType atomicType = AtomicType::AtomicNone,
          ReluPreMode reluPreMode = ReluPreMode::NoRelu,
          typename = std::enable_if_t<is_tile_data_v<FpTileData> && (FpTileData::Loc == TileType::Scaling || FpTileData::Loc == TileType::Vec) &&
                                      sizeof(typename FpTileData::DType) == 8>>
PTO_INST RecordEvent TSTORE(GlobalData& dst, TileData& src, FpTileData& fp)
{
    PTO_AMD_TRACE_INSTR(1, TR_TSTORE_FP, dst, src, fp);
    static_assert(atomicType == AtomicType::AtomicNone, "the quantising TSTORE does not add atomically");
    const uint8_t* words = fp.Storage();
    const auto word_of = [&](int col) { return *reinterpret_cast<const uint64_t*>(words + fp.ByteOffset(0, col)); };
    if constexpr (TileData::Loc == TileType::Acc)
        amd::tstore_acc_quant<true, TileData, GlobalData, reluPreMode>(dst, src, word_of);
    else
        amd::tstore_lds_quant<true, TileData, GlobalData, reluPreMode>(dst, src, word_of);
    return {};
}

template <typename TileData, typename GlobalData, typename FpTileData, AtomicType atomicType = AtomicType::AtomicNone,
          ReluPreMode reluPreMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<is_tile_data_v<FpTileData> && all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TSTORE_FP(GlobalData& dst, TileData& src, FpTileData& fp, WaitEvents&...)
{
    return TSTORE<TileData, GlobalData, FpTileData, atomicType, reluPreMode>(dst, src, fp);
}

// ---- TMOV / TEXTRACT -----------------------------------------------------------------------------------------------
namespace amd {
// Accumulator -> on-chip buffer tile, the fix-pipe move: dst(r, c) = f(src(r + row0, c + col0)) over dst's valid region
// (reference: cpu/TExtract.hpp:21-46).  QUANT 0: optional relu, then the element conversion of TSTORE; 1 / 2: fix-pipe
// quantisation with one word for the tile / one word per source column (cpu/common.hpp:139-185), relu after it.
template <int QUANT, ReluPreMode relu, typename DstTile, typename SrcTile, typename WordOf>
PTO_INST void tmov_acc(DstTile& dst, SrcTile& src, int row0, int col0, WordOf&& word_of)
{
    static_assert(DstTile::Loc == TileType::Vec || DstTile::Loc == TileType::Mat, "an accumulator tile moves to a Vec or Mat tile");
    using D = typename DstTile::DType;
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    uint8_t* d = dst.Storage();
    const bool sat_inf = QUANT != 0 && ((get_task_cookie() >> 48) & 1u);
    __syncthreads();
    for_each_acc(src, [&](int slot, int r, int row, int col) {
        const int dr = row - row0, dc = col - col0;
        if (dr >= 0 && dc >= 0 && dr < vr && dc < vc && row < src.GetValidRow() && col < src.GetValidCol()) {
            if constexpr (QUANT == 0) {
                auto v = src.regs[slot][r];
                if constexpr (relu == ReluPreMode::NormalRelu)
                    v = v > 0 ? v : 0;
                *reinterpret_cast<D*>(d + dst.ByteOffset(dr, dc)) = convert<D>(v);
            } else {
                float v = quantize_element<QUANT == 2, D>(src.regs[slot][r], word_of(col), sat_inf);
                if constexpr (relu == ReluPreMode::NormalRelu)
                    v = v > 0 ? v : 0;
                *reinterpret_cast<D*>(d + dst.ByteOffset(dr, dc)) = static_cast<D>(v);
            }
        }
    });
    __syncthreads();
}
// Into an accumulator tile: dst(r, c) = src(r + row0, c + col0) over dst's valid region, element by element with the
// reference's implicit conversion (cpu/TMov.hpp:28-33, cpu/TExtract.hpp:21-46; the simulator places no restriction on
// the destination).  From another accumulator of the same shape the move is register to register; from an on-chip
// buffer tile every lane fetches the elements of the blocks it holds.  Elements outside the valid region keep their value.
template <ReluPreMode relu, typename DstTile, typename SrcTile>
PTO_INST void tmov_into_acc(DstTile& dst, SrcTile& src, int row0, int col0)
{
    using Reg = typename DstTile::Reg;
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    if constexpr (SrcTile::Loc == TileType::Acc) {
        static_assert(DstTile::Rows == SrcTile::Rows && DstTile::Cols == SrcTile::Cols,
                      "accumulator to accumulator moves keep the tile shape (registers do not change lanes)");
        for_each_acc(dst, [&](int slot, int r, int row, int col) {
            if (row < vr && col < vc) {
                Reg v = static_cast<Reg>(src.regs[slot][r]);
                if constexpr (relu == ReluPreMode::NormalRelu)
                    v = v > 0 ? v : 0;
                dst.regs[slot][r] = v;
            }
        });
    } else {
        using S = typename SrcTile::DType;
        acquire(src);
        __syncthreads();  // writers of the source tile are done
        const uint8_t* ps = src.Storage();
        for_each_acc(dst, [&](int slot, int r, int row, int col) {
            if (row < vr && col < vc) {
                Reg v = static_cast<Reg>(*reinterpret_cast<const S*>(ps + src.ByteOffset(row + row0, col + col0)));
                if constexpr (relu == ReluPreMode::NormalRelu)
                    v = v > 0 ? v : 0;
                dst.regs[slot][r] = v;
            }
        });
    }
}
// relu over the valid region of an LDS tile (TMOV's relu form between buffer tiles, cpu/TMov.hpp:37-54)
template <typename TileData>
PTO_INST void trelu_lds(TileData& t)
{
    using T = typename TileData::DType;
    static_assert(is_number<T>, "relu needs a numeric element type");
    const int vr = t.GetValidRow(), vc = t.GetValidCol();
    uint8_t* d = t.Storage();
    for (int idx = threadIdx.x; idx < vr * vc; idx += PTO_AMD_THREADS) {
        const int r = idx / vc, c = idx - r * vc;
        T* e = reinterpret_cast<T*>(d + t.ByteOffset(r, c));
        if (*e < T(0))
            *e = T(0);
    }
    __syncthreads();
}
}  // namespace amd

template <typename DstTileData, typename SrcTileData, ReluPreMode reluMode, typename... WaitEvents,
          std::enable_if_t<all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TMOV(DstTileData& dst, SrcTileData& src, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMOV, dst, src);
    if constexpr (DstTileData::Loc == TileType::Acc) {
        amd::tmov_into_acc<reluMode>(dst, src, 0, 0);
    } else if constexpr (SrcTileData::Loc == TileType::Acc) {
        amd::tmov_acc<0, reluMode>(dst, src, 0, 0, [](int) { return (uint64_t)0; });
    } else {
        amd::textract_lds<reluMode == ReluPreMode::NoRelu>(dst, src, 0, 0);
        if constexpr (reluMode == ReluPreMode::NormalRelu)
            amd::trelu_lds(dst);
    }
    return {};
}
template <typename DstTileData, typename SrcTileData, typename... WaitEvents, std::enable_if_t<all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TMOV(DstTileData& dst, SrcTileData& src, WaitEvents&...)
{
    return TMOV<DstTileData, SrcTileData, ReluPreMode::NoRelu>(dst, src);
}
// fix-pipe quantising forms: one scalar word, or one word per column from a Scaling tile
template <typename DstTileData, typename SrcTileData, ReluPreMode reluMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TMOV(DstTileData& dst, SrcTileData& src, uint64_t preQuantScalar, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMOV, dst, src);
    static_assert(SrcTileData::Loc == TileType::Acc, "the quantising TMOV drains an accumulator tile");
    amd::tmov_acc<1, reluMode>(dst, src, 0, 0, [&](int) { return preQuantScalar; });
    return {};
}
template <typename DstTileData, typename SrcTileData, typename FpTileData, ReluPreMode reluMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<is_tile_data_v<FpTileData> && FpTileData::Loc == TileType::Scaling && all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TMOV(DstTileData& dst, SrcTileData& src, FpTileData& fp, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMOV, dst, src, fp);
    static_assert(SrcTileData::Loc == TileType::Acc, "the quantising TMOV drains an accumulator tile");
    static_assert(sizeof(typename FpTileData::DType) == 8, "the Scaling tile holds one 64-bit quantisation word per column");
    const uint8_t* words = fp.Storage();
    amd::tmov_acc<2, reluMode>(dst, src, 0, 0, [&](int col) { return *reinterpret_cast<const uint64_t*>(words + fp.ByteOffset(0, col)); });
    return {};
}

template <typename DstTileData, typename SrcTileData, ReluPreMode reluMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TEXTRACT(DstTileData& dst, SrcTileData& src, uint16_t indexRow = 0, uint16_t indexCol = 0, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TEXTRACT, dst, src);
    static_assert(DstTileData::Loc != TileType::Acc || SrcTileData::Loc != TileType::Acc,
                  "TEXTRACT between accumulator tiles would move registers across lanes: go through a Vec tile");
    if constexpr (DstTileData::Loc == TileType::Acc) {
        amd::tmov_into_acc<reluMode>(dst, src, indexRow, indexCol);
    } else if constexpr (SrcTileData::Loc == TileType::Acc) {
        amd::tmov_acc<0, reluMode>(dst, src, indexRow, indexCol, [](int) { return (uint64_t)0; });
    } else {
        amd::textract_lds<reluMode == ReluPreMode::NoRelu>(dst, src, indexRow, indexCol);
        if constexpr (reluMode == ReluPreMode::NormalRelu)
            amd::trelu_lds(dst);
    }
    return {};
}
template <typename DstTileData, typename SrcTileData, ReluPreMode reluMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TEXTRACT(DstTileData& dst, SrcTileData& src, uint64_t preQuantScalar, uint16_t indexRow, uint16_t indexCol, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TEXTRACT, dst, src);
    static_assert(SrcTileData::Loc == TileType::Acc, "the quantising TEXTRACT drains an accumulator tile");
    amd::tmov_acc<1, reluMode>(dst, src, indexRow, indexCol, [&](int) { return preQuantScalar; });
    return {};
}
template <typename DstTileData, typename SrcTileData, typename FpTileData, ReluPreMode reluMode = ReluPreMode::NoRelu, typename... WaitEvents,
          std::enable_if_t<is_tile_data_v<FpTileData> && FpTileData::Loc == TileType::Scaling && all_events_v<WaitEvents...>, int> = 0>
PTO_INST RecordEvent TEXTRACT(DstTileData& dst, SrcTileData& src, FpTileData& fp, uint16_t indexRow, uint16_t indexCol, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TEXTRACT, dst, src, fp);
    static_assert(SrcTileData::Loc == TileType::Acc, "the quantising TEXTRACT drains an accumulator tile");
    static_assert(sizeof(typename FpTileData::DType) == 8, "the Scaling tile holds one 64-bit quantisation word per column");
    const uint8_t* words = fp.Storage();
    amd::tmov_acc<2, reluMode>(dst, src, indexRow, indexCol,
                               [&](int col) { return *reinterpret_cast<const uint64_t*>(words + fp.ByteOffset(0, col)); });
    return {};
}

// ---- TMATMUL family ------------------------------------------------------------------------------------------------
namespace amd {
template <typename TileRes>
PTO_INST void copy_acc(TileRes& out, TileRes& in)
{
    if (&out != &in) {
#pragma unroll
        for (int s = 0; s < TileRes::NBLK; ++s)
            out.regs[s] = in.regs[s];
    }
}
// bias (1 x N, any LDS tile) is added after the K loop, per column (reference: cpu/TMatmul.hpp:219-230)
template <typename TileRes, typename TileBias>
PTO_INST void add_bias_row(TileRes& c, TileBias& bias)
{
    using B = typename TileBias::DType;
    const uint8_t* pb = bias.Storage();
    const int vc = c.GetValidCol();
    for_each_acc(c, [&](int slot, int r, int, int col) {
        if (col < vc)
            c.regs[slot][r] += static_cast<typename TileRes::Reg>(*reinterpret_cast<const B*>(pb + bias.ByteOffset(0, col)));
    });
}
}  // namespace amd

template <typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TMATMUL(TileRes& cMatrix, TileLeftT& aMatrix, TileRightT& bMatrix, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMATMUL, cMatrix, aMatrix, bMatrix);
    amd::tmatmul<true>(cMatrix, aMatrix, bMatrix);
    return {};
}
template <AccPhase Phase, typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TMATMUL(TileRes& cMatrix, TileLeftT& aMatrix, TileRightT& bMatrix, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMATMUL, cMatrix, aMatrix, bMatrix);
    amd::tmatmul<true>(cMatrix, aMatrix, bMatrix);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TMATMUL_ACC(TileRes& cOutMatrix, TileRes& cInMatrix, TileLeftT& aMatrix, TileRightT& bMatrix, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMATMUL_ACC, cOutMatrix, cInMatrix, aMatrix, bMatrix);
    amd::copy_acc(cOutMatrix, cInMatrix);
    amd::tmatmul<false>(cOutMatrix, aMatrix, bMatrix);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TMATMUL_ACC(TileRes& cMatrix, TileLeftT& aMatrix, TileRightT& bMatrix, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMATMUL_ACC, cMatrix, cMatrix, aMatrix, bMatrix);
    amd::tmatmul<false>(cMatrix, aMatrix, bMatrix);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileRightT, typename TileBias, typename... WaitEvents>
PTO_INST RecordEvent TMATMUL_BIAS(TileRes& cMatrix, TileLeftT& aMatrix, TileRightT& bMatrix, TileBias& biasData, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TMATMUL_BIAS, cMatrix, aMatrix, bMatrix, biasData);
    amd::tmatmul<true>(cMatrix, aMatrix, bMatrix);
    amd::add_bias_row(cMatrix, biasData);
    return {};
}
// ---- TMATMUL_MX / TGEMV_MX (fp8 E4M3 / E5M2 or fp4 E2M1 operands; reference: cpu/TMatmul.hpp:169-205,254-326) ------------------
// (a trace record names the accumulator and the two operand tiles; the scale tiles follow their operands)
namespace amd {
template <TraceOpOrInt OP, typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT>
PTO_INST void tmatmul_mx_plain(TileRes& c, TileLeftT& a, TileLeftScaleT& as, TileRightT& b, TileRightScaleT& bs)
{
    PTO_AMD_TRACE_INSTR(1, PTO_AMD_TRACE_OP(OP), c, a, b);
    tmatmul_mx<true>(c, a, as, b, bs);
}
template <TraceOpOrInt OP, typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT>
PTO_INST void tmatmul_mx_acc(TileRes& cOut, TileRes& cIn, TileLeftT& a, TileLeftScaleT& as, TileRightT& b, TileRightScaleT& bs)
{
    PTO_AMD_TRACE_INSTR(1, PTO_AMD_TRACE_OP(OP), cOut, cIn, a, b);
    copy_acc(cOut, cIn);
    tmatmul_mx<false>(cOut, a, as, b, bs);
}
template <TraceOpOrInt OP, typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT, typename TileBias>
PTO_INST void tmatmul_mx_bias(TileRes& c, TileLeftT& a, TileLeftScaleT& as, TileRightT& b, TileRightScaleT& bs, TileBias& bias)
{
    static_assert(std::is_same_v<typename TileBias::DType, float> && TileBias::Rows == 1, "TMATMUL_MX: bias is one row of float");
    PTO_AMD_TRACE_INSTR(1, PTO_AMD_TRACE_OP(OP), c, a, b, bias);
    tmatmul_mx<true>(c, a, as, b, bs);
    add_bias_row(c, bias);
}
}  // namespace amd
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft>>
PTO_INST RecordEvent TMATMUL_MX(TileRes& cMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale, TileRightT& bMatrix, TileRightScaleT& bScale)
{
    amd::tmatmul_mx_plain<PTO_AMD_TR(TR_TMATMUL_MX)>(cMatrix, aMatrix, aScale, bMatrix, bScale);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft>>
PTO_INST RecordEvent TMATMUL_MX(TileRes& cOutMatrix, TileRes& cInMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale,
                                TileRightT& bMatrix, TileRightScaleT& bScale)
{
    amd::tmatmul_mx_acc<PTO_AMD_TR(TR_TMATMUL_MX)>(cOutMatrix, cInMatrix, aMatrix, aScale, bMatrix, bScale);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT, typename TileBias,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft && TileBias::Loc == TileType::Bias>>
PTO_INST RecordEvent TMATMUL_MX(TileRes& cMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale, TileRightT& bMatrix,
                                TileRightScaleT& bScale, TileBias& biasData)
{
    amd::tmatmul_mx_bias<PTO_AMD_TR(TR_TMATMUL_MX)>(cMatrix, aMatrix, aScale, bMatrix, bScale, biasData);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft>>
PTO_INST RecordEvent TGEMV_MX(TileRes& cMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale, TileRightT& bMatrix, TileRightScaleT& bScale)
{
    amd::tmatmul_mx_plain<PTO_AMD_TR(TR_TGEMV_MX)>(cMatrix, aMatrix, aScale, bMatrix, bScale);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft>>
PTO_INST RecordEvent TGEMV_MX(TileRes& cOutMatrix, TileRes& cInMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale, TileRightT& bMatrix,
                              TileRightScaleT& bScale)
{
    amd::tmatmul_mx_acc<PTO_AMD_TR(TR_TGEMV_MX)>(cOutMatrix, cInMatrix, aMatrix, aScale, bMatrix, bScale);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileLeftScaleT, typename TileRightT, typename TileRightScaleT, typename TileBias,
          typename = std::enable_if_t<TileLeftScaleT::Loc == TileType::ScaleLeft && TileBias::Loc == TileType::Bias>>
PTO_INST RecordEvent TGEMV_MX(TileRes& cMatrix, TileLeftT& aMatrix, TileLeftScaleT& aScale, TileRightT& bMatrix, TileRightScaleT& bScale,
                              TileBias& biasData)
{
    amd::tmatmul_mx_bias<PTO_AMD_TR(TR_TGEMV_MX)>(cMatrix, aMatrix, aScale, bMatrix, bScale, biasData);
    return {};
}

template <typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TGEMV(TileRes& c, TileLeftT& a, TileRightT& b, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TGEMV, c, a, b);
    amd::tmatmul<true>(c, a, b);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileRightT, typename... WaitEvents>
PTO_INST RecordEvent TGEMV_ACC(TileRes& cOut, TileRes& cIn, TileLeftT& a, TileRightT& b, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TGEMV_ACC, cOut, cIn, a, b);
    amd::copy_acc(cOut, cIn);
    amd::tmatmul<false>(cOut, a, b);
    return {};
}
template <typename TileRes, typename TileLeftT, typename TileRightT, typename TileBias, typename... WaitEvents>
PTO_INST RecordEvent TGEMV_BIAS(TileRes& c, TileLeftT& a, TileRightT& b, TileBias& bias, WaitEvents&...)
{
    PTO_AMD_TRACE_INSTR(1, TR_TGEMV_BIAS, c, a, b, bias);
    amd::tmatmul<true>(c, a, b);
    amd::add_bias_row(c, bias);
    return {};
}

}  // namespace pto

// wait_flag(PIPE_MTE2, PIPE_MTE1, id, tiles...): the reference's "the loads have arrived" flag, given the Mat tiles it
// stands for.  Plain wait_flag orders nothing here (every instruction waits for what it reads); this form lets a kernel
// wait for the asynchronous TLOADs of several tiles with one barrier, in the place where the reference program has its
// wait_flag(PIPE_MTE2, PIPE_MTE1, ...) (kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp:131-136).
template <typename... Tiles, typename = std::enable_if_t<(sizeof...(Tiles) > 0)>>
PTO_INST void wait_flag(pto::pipe_t, pto::pipe_t, pto::event_t, Tiles&... tiles)
{
    pto::amd::acquire_all(tiles...);
}
