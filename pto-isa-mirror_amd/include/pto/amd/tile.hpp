// Tile<>: a 2-D on-chip operand.  Reference: include/pto/common/pto_tile.hpp:1422-1835 (template parameters, aliases,
// valid-shape accessors), cpu/TAssign.hpp:21-36 (address binding).
//
// Where a tile lives on gfx950:
//   Vec (UB), Bias, Scaling, ScaleLeft/Right, Mat without a box layout : LDS, plain row-major [Rows][Cols]
//   Mat (L1) with a box layout : LDS, "lines" of contiguous elements with the 16-byte chunks of a line XOR-swizzled by
//                the line index: SLayout::RowMajor boxes (NZ, the A-side panels) keep rows as lines, [Rows][Cols];
//                SLayout::ColMajor boxes (ZN, the B-side panels) keep columns as lines, [Cols][Rows].  Either way a
//                GEMM panel is stored K-contiguous, which is what a 16-byte global -> LDS copy delivers and what an
//                MFMA fragment read wants (packed fp4 Mat tiles stay plain row-major)
//   Left  (L0A) : lines = rows, [M][K]; Right (L0B) : lines = columns, [N][K]; same swizzle.  A Left / Right tile is
//                either a window onto the Mat tile it was extracted from (no bytes move: the matrix unit is fed from
//                LDS through registers, there is no separate L0 memory to fill) or, when the extraction cannot be a
//                window (unaligned offsets, ragged valid regions, a transposing or re-pairing move), a copy in the
//                L0A / L0B region.  A window is valid until its Mat tile is next written.
//   Acc   (L0C) : registers; the tile is cut into 32 x 32 MFMA blocks; when the block grid divides over a grid of
//                waves each wave owns a rectangle of blocks (so an operand fragment feeds several MFMAs), otherwise
//                block b belongs to wave b % WAVES
// BLayout / SLayout / fractal size select among these; the internal layouts are the backend's own (they are invisible
// in global-memory results).
#pragma once
#include "base.hpp"

namespace pto {
namespace amd {

constexpr int WAVES = PTO_AMD_THREADS / 64;

// the core's LDS arena and its regions
__device__ __forceinline__ uint8_t* lds_arena()
{
    extern __shared__ __align__(16) uint8_t pto_amd_lds[];
    return pto_amd_lds;
}
template <TileType L>
struct Region {
    static constexpr bool in_lds = L != TileType::Acc && L != TileType::Ctrl;
    static constexpr uint32_t L1 = 0, L0A = L1 + PTO_AMD_L1_BYTES, L0B = L0A + PTO_AMD_L0A_BYTES, UB = L0B + PTO_AMD_L0B_BYTES,
                              BT = UB + PTO_AMD_UB_BYTES, FB = BT + PTO_AMD_BIAS_BYTES, L0S = FB + PTO_AMD_FB_BYTES;
    static constexpr uint32_t base = L == TileType::Mat          ? L1
                                     : L == TileType::Left       ? L0A
                                     : L == TileType::Right      ? L0B
                                     : L == TileType::Vec        ? UB
                                     : L == TileType::Bias       ? BT
                                     : L == TileType::Scaling    ? FB
                                     : L == TileType::ScaleLeft  ? L0S
                                                                 : L0S + PTO_AMD_L0S_BYTES / 2;  // ScaleRight
    static constexpr uint32_t size = L == TileType::Mat       ? PTO_AMD_L1_BYTES
                                     : L == TileType::Left    ? PTO_AMD_L0A_BYTES
                                     : L == TileType::Right   ? PTO_AMD_L0B_BYTES
                                     : L == TileType::Vec     ? PTO_AMD_UB_BYTES
                                     : L == TileType::Bias    ? PTO_AMD_BIAS_BYTES
                                     : L == TileType::Scaling ? PTO_AMD_FB_BYTES
                                                              : PTO_AMD_L0S_BYTES / 2;
};
// The fix-pipe staging bytes follow the regions -- or, with PTO_AMD_STAGE_IN_L1 defined, lie over the start of L1: a
// kernel whose L1 tiles are dead by the time it stores (the usual GEMM shape) then needs no LDS for them; TSTORE puts a
// workgroup barrier in front of its first staging write so that every wave is done reading L1.
constexpr uint32_t REGIONS_END = PTO_AMD_L1_BYTES + PTO_AMD_L0A_BYTES + PTO_AMD_L0B_BYTES + PTO_AMD_UB_BYTES +
                                 PTO_AMD_BIAS_BYTES + PTO_AMD_FB_BYTES + PTO_AMD_L0S_BYTES;
#ifdef PTO_AMD_STAGE_IN_L1
constexpr bool STAGE_ALIASES_L1 = true;
constexpr uint32_t STAGE_BASE = 0;
constexpr uint32_t LDS_TOTAL = REGIONS_END;
static_assert(PTO_AMD_STAGE_BYTES <= PTO_AMD_L1_BYTES, "the staging bytes lie inside L1");
#else
constexpr bool STAGE_ALIASES_L1 = false;
constexpr uint32_t STAGE_BASE = REGIONS_END;
constexpr uint32_t LDS_TOTAL = STAGE_BASE + PTO_AMD_STAGE_BYTES;
#endif
#ifndef PTO_AMD_CHECK_REFERENCE_SOURCE
static_assert(LDS_TOTAL <= 160 * 1024, "the on-chip regions must fit the 160 KiB LDS of a CU");
#endif

// Sticky status word of the kernels of this translation unit: 0, or the first constraint a core violated
// (1: TASSIGN address outside its region, 2: TQUANT NZ mode on a tile that is not whole 16-row x 2-group boxes).
// pto::amd::device_status() reads it on the host.
static __device__ int g_status = 0;
// The task cookie of this translation unit's cores (reference: get_task_cookie(), common/cpu_stub.hpp:606-612): control
// bits the fix-pipe consults; bit 48 = saturate non-finite results of the half / bfloat16 quantising drains
// (cpu/common.hpp:143-171).  pto::amd::set_task_cookie() writes it from the host.
static __device__ unsigned long long g_task_cookie = 0;
__device__ __forceinline__ uint64_t get_task_cookie() { return g_task_cookie; }
__device__ __forceinline__ void report(int code)
{
    if (threadIdx.x == 0)
        atomicCAS(&g_status, 0, code);
}

template <typename T>
struct ElemTraits {
    static constexpr int bytes2 = 2 * (int)sizeof(T);  // bytes of two elements
};
template <>
struct ElemTraits<float4_e2m1x2_t> {
    static constexpr int bytes2 = 1;
};
template <>
struct ElemTraits<float4_e1m2x2_t> {
    static constexpr int bytes2 = 1;
};

// ---- swizzled line storage ---------------------------------------------------------------------------------------------
// A line of LINE_BYTES bytes holds 16-byte chunks; chunk c of line l is stored at chunk position c ^ ((l >> sh) & mask).
// sh / mask are chosen so that 16 consecutive lines read at one chunk index -- what a quarter wave of ds_read_b128 does
// when it fetches MFMA fragments -- touch 16 different 16-byte slots of the 256 bytes that span all LDS banks:
//   2 chunks per line (32 B): 8 lines per 256 B, lines l and l + 8 differ in the chunk bit     sh 3, mask 1
//   4 chunks (64 B) sh 2, mask 3;   8 chunks (128 B) sh 1, mask 7;   16 or more chunks sh 0, mask 15
template <int LINE_BYTES>
struct LineSwizzle {
    static constexpr int chunks = LINE_BYTES / 16;
    static constexpr bool on = LINE_BYTES % 16 == 0 && chunks >= 2 && (chunks & (chunks - 1)) == 0;
    static constexpr uint32_t sh = !on ? 0 : (chunks >= 16 ? 0 : (chunks == 8 ? 1 : (chunks == 4 ? 2 : 3)));
    static constexpr uint32_t mask = !on ? 0 : (chunks >= 16 ? 15 : (uint32_t)chunks - 1);
};
PTO_INST uint32_t line_offset(uint32_t line, uint32_t kbyte, uint32_t pitch, uint32_t sh, uint32_t mask)
{
    return line * pitch + ((((kbyte >> 4) ^ ((line >> sh) & mask)) << 4) | (kbyte & 15u));
}

// how the accumulator blocks of an RB x CB block grid are dealt to the waves: a WR x WC grid of waves, each owning
// (RB / WR) x (CB / WC) neighbouring blocks, with the split that needs the fewest operand fragments per k-step;
// WR = 0 when no split divides the grid (blocks are then dealt round-robin)
struct WaveGrid {
    int wr, wc;
};
constexpr WaveGrid pick_wave_grid(int rb, int cb, int waves)
{
    WaveGrid best{0, 0};
    int best_cost = 1 << 30;
    for (int wr = 1; wr <= waves; ++wr) {
        if (waves % wr != 0)
            continue;
        const int wc = waves / wr;
        if (rb % wr != 0 || cb % wc != 0)
            continue;
        const int cost = rb / wr + cb / wc;
        if (cost < best_cost) {
            best_cost = cost;
            best = WaveGrid{wr, wc};
        }
    }
    return best;
}

// register storage of an accumulator tile.  Blocks are kept transposed: lane (l32, lhi) of the owning wave holds row
// l32 of the block and, in register r, column 8 (r / 4) + 4 lhi + r % 4 -- four consecutive columns per register quad,
// so a drain to row-major memory writes 8 or 16 contiguous bytes per lane and quad.
template <typename T, int Rows, int Cols>
struct AccStorage {
    static constexpr int RB = (Rows + 31) / 32, CB = (Cols + 31) / 32;
    static constexpr WaveGrid grid = pick_wave_grid(RB, CB, WAVES);
    static constexpr bool BLOCKED = grid.wr != 0;
    static constexpr int MB = BLOCKED ? RB / grid.wr : 1, NB = BLOCKED ? CB / grid.wc : 1;
    static constexpr int NBLK = BLOCKED ? MB * NB : (RB * CB + WAVES - 1) / WAVES;
    using Reg = std::conditional_t<std::is_integral_v<T>, int32_t, float>;
    typedef Reg Vec16 __attribute__((ext_vector_type(16)));
    Vec16 regs[NBLK];
    // block (bi, bj) held in slot `slot` of wave `wave`; false when the slot is empty (round-robin dealing only)
    PTO_INST static bool block_of(int slot, int wave, int& bi, int& bj)
    {
        if constexpr (BLOCKED) {
            bi = (wave / grid.wc) * MB + slot / NB;
            bj = (wave % grid.wc) * NB + slot % NB;
            return true;
        } else {
            const int blk = slot * WAVES + wave;
            bi = blk / CB;
            bj = blk - bi * CB;
            return blk < RB * CB;
        }
    }
};
struct LdsStorage {
    uint32_t lds_ = 0;   // byte offset of the tile in the arena
    uint32_t addr_ = 0;  // the TASSIGN address (offset inside the tile's region)
    uint32_t pend_ = 0;  // Mat tiles: an asynchronous TLOAD into the tile may still be in flight
};
// The tiles the matrix unit reads -- Left / Right and their scale tiles -- are stored as lines along K (rows of the A
// side, columns of the B side) and may be windows onto a Mat tile instead of owning bytes.
constexpr bool is_operand_loc(TileType l)
{
    return l == TileType::Left || l == TileType::Right || l == TileType::ScaleLeft || l == TileType::ScaleRight;
}
// Left / Right / ScaleLeft / ScaleRight tiles: where the lines live (the tile's own storage, or a window onto a Mat tile)
struct WindowStorage : LdsStorage {
    uint32_t pitch_ = 0, sh_ = 0, mask_ = 0;  // line pitch in bytes and the swizzle of the storage the lines live in
    uint32_t line0_ = 0, kb0_ = 0;            // first line / first byte along a line of the window
    uint32_t own_ok_ = 1;                     // the tile's own storage lies inside its region (needed by copies only)
};

}  // namespace amd

template <TileType Loc_, typename Element_, const int Rows_, const int Cols_, const BLayout BFractal_ = BLayout::RowMajor,
          const int RowValid_ = Rows_, const int ColValid_ = Cols_, const SLayout SFractal_ = SLayout::NoneBox,
          const int SFractalSize_ = TileConfig::fractalABSize, auto PadVal_ = PadValue::Null,
          const CompactMode Compact_ = CompactMode::Null>
struct Tile : std::conditional_t<Loc_ == TileType::Acc, amd::AccStorage<Element_, Rows_, Cols_>,
                                 std::conditional_t<amd::is_operand_loc(Loc_), amd::WindowStorage, amd::LdsStorage>> {
    using DType = Element_;
    static constexpr TileType Loc = Loc_;
    static constexpr int Rows = Rows_, Cols = Cols_, ValidRow = RowValid_, ValidCol = ColValid_;
    static constexpr BLayout BFractal = BFractal_;
    static constexpr SLayout SFractal = SFractal_;
    static constexpr int SFractalSize = SFractalSize_;
    static constexpr auto PadVal = PadVal_;
    static constexpr CompactMode Compact = Compact_;
    static constexpr int Numel = Rows_ * Cols_;
    static constexpr uint32_t Bytes = (uint32_t)((int64_t)Rows_ * Cols_ * amd::ElemTraits<Element_>::bytes2 / 2);
    static constexpr bool isRowMajor = BFractal_ == BLayout::RowMajor;

    int vrow_ = RowValid_, vcol_ = ColValid_;

    // a tile that was never TASSIGNed sits at the start of its own region (not of the arena, which is L1)
    PTO_INST Tile() { BindDefault(); }
    // dynamic valid extents, in declaration order (reference: pto_tile.hpp:1654-1676)
    PTO_INST Tile(int a)
    {
        BindDefault();
        if constexpr (RowValid_ == DYNAMIC)
            vrow_ = a;
        else
            vcol_ = a;
    }
    PTO_INST Tile(int r, int c) : vrow_(r), vcol_(c) { BindDefault(); }
    // ---- storage layout (static part) ----
    static constexpr bool is_packed4 = amd::ElemTraits<Element_>::bytes2 == 1;
    // Mat tiles with a box layout are stored as swizzled lines; lines are rows for SLayout::RowMajor boxes, columns for
    // SLayout::ColMajor boxes
    // (a line of packed fp4 codes keeps the two codes of a byte neighbours along the line)
    static constexpr bool MatLines = Loc_ == TileType::Mat && SFractal_ != SLayout::NoneBox;
    static constexpr bool OperandLoc = amd::is_operand_loc(Loc_);
    static constexpr bool Lined = MatLines || OperandLoc;
    static constexpr bool LinesAreRows = Loc_ == TileType::Left || Loc_ == TileType::ScaleLeft || (MatLines && SFractal_ == SLayout::RowMajor);
    static constexpr int Lines = LinesAreRows ? Rows_ : Cols_;
    static constexpr int LineBytes = (LinesAreRows ? Cols_ : Rows_) * amd::ElemTraits<Element_>::bytes2 / 2;
    using Swz = amd::LineSwizzle<LineBytes>;

    PTO_INST void BindDefault()
    {
        if constexpr (Loc_ != TileType::Acc)
            this->lds_ = amd::Region<Loc_>::base;
        if constexpr (OperandLoc) {
            this->own_ok_ = Bytes <= amd::Region<Loc_>::size;
            BindOwnLines();
        }
    }
    // the lines are the tile's own storage (not a window onto a Mat tile)
    PTO_INST void BindOwnLines()
    {
        if constexpr (OperandLoc) {
            this->lds_ = amd::Region<Loc_>::base + this->addr_;
            this->pitch_ = LineBytes;
            this->sh_ = Swz::sh;
            this->mask_ = Swz::mask;
            this->line0_ = 0;
            this->kb0_ = 0;
        }
    }
    static constexpr size_t GetSizeInBytes() { return Bytes; }
    PTO_INST int GetValidRow() const { return vrow_; }
    PTO_INST int GetValidCol() const { return vcol_; }

    // byte offset of logical element (r, c) inside the tile's LDS storage (fp4: of the byte holding it)
    PTO_INST uint32_t ByteOffset(int r, int c) const
    {
        constexpr int b2 = amd::ElemTraits<Element_>::bytes2;
        if constexpr (OperandLoc) {
            const uint32_t line = (uint32_t)(LinesAreRows ? r : c) + this->line0_;
            const uint32_t kb = (uint32_t)((LinesAreRows ? c : r) * b2 / 2) + this->kb0_;
            return amd::line_offset(line, kb, this->pitch_, this->sh_, this->mask_);
        } else if constexpr (MatLines) {
            return amd::line_offset((uint32_t)(LinesAreRows ? r : c), (uint32_t)((LinesAreRows ? c : r) * b2 / 2), LineBytes, Swz::sh,
                                    Swz::mask);
        } else {
            return (uint32_t)(((int64_t)r * Cols_ + c) * b2 / 2);
        }
    }
    // which nibble of that byte holds element (r, c) of a packed fp4 tile: the two codes of a byte are neighbours along a
    // line where the tile is stored as lines (down a column for Right tiles and column-lined Mat tiles), along a row
    // otherwise
    static constexpr bool PairsDownColumns = Loc_ == TileType::Right || (MatLines && !LinesAreRows);
    PTO_INST static int Nibble(int r, int c) { return PairsDownColumns ? (r & 1) : (c & 1); }
    // the tile's on-chip address as TASSIGN bound it (what the reference's data() pointer stands for)
    PTO_INST uint64_t data() const
    {
        if constexpr (Loc_ == TileType::Acc)
            return 0;
        else
            return this->addr_;
    }
    PTO_INST uint8_t* Storage() const
    {
        static_assert(Loc_ != TileType::Acc, "accumulator tiles live in registers");
        return amd::lds_arena() + this->lds_;
    }
};

template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileLeft = Tile<TileType::Left, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_, SLayout::RowMajor,
                      TileConfig::fractalABSize>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileRight = Tile<TileType::Right, Element_, Rows_, Cols_, BLayout::RowMajor, RowValid_, ColValid_, SLayout::ColMajor,
                       TileConfig::fractalABSize>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileAcc = Tile<TileType::Acc, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_, SLayout::RowMajor,
                     TileConfig::fractalCSize>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileLeftScale = Tile<TileType::ScaleLeft, Element_, Rows_, Cols_, BLayout::RowMajor, RowValid_, ColValid_,
                           SLayout::RowMajor, TileConfig::fractalMxSize>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileRightScale = Tile<TileType::ScaleRight, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_,
                            SLayout::ColMajor, TileConfig::fractalMxSize>;

// the Compact forms (reference: common/pto_tile.hpp:1780-1835): same tiles, CompactMode::Normal recorded in the type
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileLeftCompact = Tile<TileType::Left, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_, SLayout::RowMajor,
                             TileConfig::fractalABSize, PadValue::Null, CompactMode::Normal>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileRightCompact = Tile<TileType::Right, Element_, Rows_, Cols_, BLayout::RowMajor, RowValid_, ColValid_, SLayout::ColMajor,
                              TileConfig::fractalABSize, PadValue::Null, CompactMode::Normal>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileAccCompact = Tile<TileType::Acc, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_, SLayout::RowMajor,
                            TileConfig::fractalCSize, PadValue::Null, CompactMode::Normal>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileLeftScaleCompact = Tile<TileType::ScaleLeft, Element_, Rows_, Cols_, BLayout::RowMajor, RowValid_, ColValid_,
                                  SLayout::RowMajor, TileConfig::fractalMxSize, PadValue::Null, CompactMode::Normal>;
template <typename Element_, const int Rows_, const int Cols_, const int RowValid_ = Rows_, const int ColValid_ = Cols_>
using TileRightScaleCompact = Tile<TileType::ScaleRight, Element_, Rows_, Cols_, BLayout::ColMajor, RowValid_, ColValid_,
                                   SLayout::ColMajor, TileConfig::fractalMxSize, PadValue::Null, CompactMode::Normal>;

template <typename T>
struct is_tile : std::false_type {};
template <TileType L, typename E, int R, int C, BLayout B, int RV, int CV, SLayout S, int F, auto P, CompactMode M>
struct is_tile<Tile<L, E, R, C, B, RV, CV, S, F, P, M>> : std::true_type {};
template <typename T>
constexpr bool is_tile_data_v = is_tile<std::remove_cv_t<T>>::value;

struct RecordEvent {};

// Instruction classes an Event orders (the subset of the reference's Op list, common/event.hpp:21-130, that the matmul
// path names).
enum class Op : uint16_t {
    TLOAD, TSTORE_VEC, SCALAR, TRESHAPE, VECTOR, TCVT, TMOV_V2V, TMOV_V2M, TEXTRACT_V2M, TMOV_M2B, TMOV_M2L, TMOV_M2R, TMOV_M2S,
    TMOV_A2V, TMOV_A2M, TSTORE_ACC, TSTORE_MAT, TMATMUL, TGEMV, TEXTRACT_M2LR, TEXTRACT_A2M, TDEQUANT, TQUANT, TFILLPAD, OP_COUNT
};
// Event<SrcOp, DstOp> (reference: common/event.hpp:361-427).  Every tile instruction of this backend is bracketed by
// workgroup barriers, so an event has nothing left to wait for: the type exists so that kernels written with explicit
// events compile and keep their meaning.  Instructions accept events as trailing arguments.
struct EventBaseTag {};
template <Op SrcOp, Op DstOp, bool AutoToken = true, event_t EventID = 0>
struct Event : EventBaseTag {
    static constexpr Op srcOp = SrcOp, dstOp = DstOp;
    PTO_INST Event() {}
    PTO_INST Event(RecordEvent) {}
    PTO_INST Event& operator=(RecordEvent) { return *this; }
    template <uint8_t CrossCoreId = 0xff>
    PTO_INST Event& Wait() { return *this; }
    template <uint8_t CrossCoreId = 0xff>
    PTO_INST Event& Init() { return *this; }
    template <uint8_t CrossCoreId = 0xff>
    PTO_INST Event& Record() { return *this; }
};
template <typename T>
struct is_event : std::is_base_of<EventBaseTag, T> {};
template <typename... Ts>
inline constexpr bool all_events_v = (is_event<Ts>::value && ...);

// address of the scale tile that belongs to a Left / Right tile at `addr` (reference: cpu/NPUMemoryModel.hpp:409-415:
// the L0 scale buffers mirror L0A / L0B at one sixteenth of the offset)
PTO_INST uint64_t GetScaleAddr(uint64_t addr) { return addr >> 4; }

// TASSIGN: binds a tile to a byte address of its on-chip buffer (reference: cpu/TAssign.hpp:21-36,
// common/pto_instr.hpp:104-121).  Accumulator tiles are register-resident: the address is accepted and ignored.
template <typename T, typename AddrType>
PTO_INST void TASSIGN(T& obj, AddrType addr)
{
    if constexpr (T::OperandLoc) {
        // a Left / Right (or scale) tile needs its own bytes only when an extraction has to copy; one that does not fit its region
        // can still be a window onto a Mat tile, so the range check is deferred to the copy
        using R = amd::Region<T::Loc>;
        uint32_t a = (uint32_t)(uint64_t)addr;
        if ((a & 15u) != 0) {
            amd::report(1);
            a = 0;
        }
        obj.addr_ = a;
        obj.own_ok_ = a + T::Bytes <= R::size;
        obj.BindOwnLines();
    } else if constexpr (T::Loc != TileType::Acc) {
        using R = amd::Region<T::Loc>;
        uint32_t a = (uint32_t)(uint64_t)addr;
        if (a + T::Bytes > R::size || (a & 15u) != 0) {
            amd::report(1);
            a = 0;
        }
        static_assert(T::Bytes <= R::size, "tile larger than its on-chip region (raise PTO_AMD_*_BYTES)");
        obj.lds_ = R::base + a;
        obj.addr_ = a;
    }
}
template <std::size_t Addr, typename T>
PTO_INST std::enable_if_t<is_tile_data_v<T>> TASSIGN(T& obj)
{
    if constexpr (T::OperandLoc) {
        static_assert(Addr % 16 == 0, "TASSIGN: address not 16-byte aligned");
    } else if constexpr (T::Loc != TileType::Acc) {
        static_assert(Addr + T::Bytes <= amd::Region<T::Loc>::size && Addr % 16 == 0,
                      "TASSIGN: address outside the tile's on-chip region or not 16-byte aligned");
    }
    TASSIGN(obj, Addr);
}

}  // namespace pto
