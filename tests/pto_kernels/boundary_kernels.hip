// PTO-style kernels for the parts of the header layer the matmul programs of matmul_kernels.hip do not reach:
// TFILLPAD and K that is not a multiple of 64 in the block-scaled matmul (program shape of
// tests/cpu/st/testcase/tmatmul_mx/tmatmul_mx_kernel.cpp:63-209, TGEMV_MX of :365-472), E1M2 operands, TCVT, TEXTRACT at
// nonzero offsets, TSTORE<AtomicAdd>, 5-D ND / DN global tensors, the fix-pipe forms of TMOV / TEXTRACT, TRESHAPE,
// Event<> / TSYNC, tiles that are never TASSIGNed, and the status word an out-of-range TASSIGN leaves behind.
// The on-chip regions are re-balanced for these programs (a larger UB for Vec tiles): the split is a compile-time
// choice of the translation unit.
#define PTO_AMD_L1_BYTES (64 * 1024)
#define PTO_AMD_L0A_BYTES (24 * 1024)
#define PTO_AMD_L0B_BYTES (24 * 1024)
#define PTO_AMD_UB_BYTES (40 * 1024)
#include <pto/pto-inst.hpp>
#include <pto/common/pto_tile.hpp>
#include <pto/common/constants.hpp>

using namespace pto;

template <typename T>
AICORE constexpr inline T CeilAlign(T a, T b)
{
    return b == 0 ? 0 : (a + b - 1) / b * b;
}

// ---- block-scaled matmul, K padded on chip -----------------------------------------------------------------------------
// A is [validM][validK], B is [validK][validN] row-major in global memory (fp4: two codes per byte); the E8M0 scales are
// the padded [M][kAlign / 32] and [kAlign / 32][N] matrices in the MX_A_ZZ / MX_B_NN layouts.  TLOAD brings the valid
// region in, TFILLPAD clears what lies beyond it, TMOV builds the Left / Right tiles.
template <typename AType, typename BType, int validM, int validK, int validN, bool isBias, bool isFp4>
__global__ AICORE void RunTMATMULMX(__gm__ float* out, __gm__ AType* src0, __gm__ BType* src1, __gm__ float8_e8m0_t* src2,
                                    __gm__ float8_e8m0_t* src3, __gm__ float* src4)
{
    using ScaleType = float8_e8m0_t;
    constexpr int blockAlign = isFp4 ? 64 : 32;
    constexpr int M = CeilAlign<int>(validM, 16);
    constexpr int kAlign = CeilAlign<int>(validK, 64);
    constexpr int N = CeilAlign<int>(validN, blockAlign);
    constexpr int kMX = kAlign / 32;

    using GlobalA = GlobalTensor<AType, Shape<1, 1, 1, validM, validK>, Stride<validM * validK, validM * validK, validM * validK, validK, 1>>;
    using GlobalB = GlobalTensor<BType, Shape<1, 1, 1, validK, validN>, Stride<validK * validN, validK * validN, validK * validN, validN, 1>>;
    using GlobalSA = GlobalTensor<ScaleType, TileShape2D<ScaleType, M, kMX, Layout::MX_A_ZZ>, BaseShape2D<ScaleType, M, kMX, Layout::MX_A_ZZ>, Layout::MX_A_ZZ>;
    using GlobalSB = GlobalTensor<ScaleType, TileShape2D<ScaleType, kMX, N, Layout::MX_B_NN>, BaseShape2D<ScaleType, kMX, N, Layout::MX_B_NN>, Layout::MX_B_NN>;
    using GlobalBias = GlobalTensor<float, Shape<1, 1, 1, 1, validN>, Stride<validN, validN, validN, validN, 1>>;
    using GlobalOut = GlobalTensor<float, Shape<1, 1, 1, validM, validN>, Stride<validM * validN, validM * validN, validM * validN, validN, 1>>;
    GlobalA aGlobal(src0);
    GlobalB bGlobal(src1);
    GlobalSA saGlobal(src2);
    GlobalSB sbGlobal(src3);
    GlobalBias biasGlobal(src4);
    GlobalOut outGlobal(out);

    using MatA = Tile<TileType::Mat, AType, M, kAlign, BLayout::ColMajor, validM, validK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, BType, kAlign, N, BLayout::ColMajor, validK, validN, SLayout::RowMajor, 512>;
    using MatSA = Tile<TileType::Mat, ScaleType, M, kMX, BLayout::RowMajor, validM, kMX, SLayout::RowMajor, 32>;
    using MatSB = Tile<TileType::Mat, ScaleType, kMX, N, BLayout::ColMajor, kMX, validN, SLayout::ColMajor, 32>;
    using MatBias = Tile<TileType::Mat, float, 1, N, BLayout::RowMajor, 1, validN>;
    MatA aMat;
    MatB bMat;
    MatSA saMat;
    MatSB sbMat;
    MatBias biasMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, M * kAlign);
    TASSIGN(saMat, M * kAlign + kAlign * N);
    TASSIGN(sbMat, M * kAlign + kAlign * N + M * kMX);
    TASSIGN(biasMat, M * kAlign + kAlign * N + M * kMX + N * kMX);

    TileLeft<AType, M, kAlign, validM, validK> aTile;
    TileRight<BType, kAlign, N, validK, validN> bTile;
    TileLeftScale<ScaleType, M, kMX, validM, kMX> saTile;
    TileRightScale<ScaleType, kMX, N, kMX, validN> sbTile;
    TileAcc<float, M, N, validM, validN> cTile;
    Tile<TileType::Bias, float, 1, N, BLayout::RowMajor, 1, validN> biasTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(biasTile, 0x0);
    TASSIGN(saTile, GetScaleAddr(aTile.data()));
    TASSIGN(sbTile, GetScaleAddr(bTile.data()));

    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    if constexpr (kAlign - validK >= blockAlign)  // (a shorter tail is inside TLOAD's own 32-byte padding)
        TFILLPAD(aMat, aMat);
    TFILLPAD(bMat, bMat);
    TLOAD<MatSA, GlobalSA>(saMat, saGlobal);
    TLOAD<MatSB, GlobalSB>(sbMat, sbGlobal);
    if constexpr (isBias)
        TLOAD(biasMat, biasGlobal);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);

    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMOV(saTile, saMat);
    TMOV(sbTile, sbMat);
    if constexpr (isBias)
        TMOV(biasTile, biasMat);
    set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
    wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);

    if constexpr (isBias)
        TMATMUL_MX(cTile, aTile, saTile, bTile, sbTile, biasTile);
    else
        TMATMUL_MX(cTile, aTile, saTile, bTile, sbTile);
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    TSTORE(outGlobal, cTile);
}

// one-row A (TGEMV_MX): the Left tile is declared a whole 512-byte row wide, B's scales come in the layout LB
template <typename AType, typename BType, int validK, int validN, Layout LB, bool isFp4>
__global__ AICORE void RunTGEMVMX(__gm__ float* out, __gm__ AType* src0, __gm__ BType* src1, __gm__ float8_e8m0_t* src2,
                                  __gm__ float8_e8m0_t* src3)
{
    using ScaleType = float8_e8m0_t;
    constexpr int blockAlign = isFp4 ? 64 : 32;
    constexpr int M = 16;
    constexpr int kAlign = CeilAlign<int>(validK, 64);
    constexpr int N = CeilAlign<int>(validN, blockAlign);
    constexpr int kMX = kAlign / 32;
    constexpr int KLeft = CeilAlign<int>(validK, isFp4 ? 1024 : 512);

    using GlobalA = GlobalTensor<AType, Shape<1, 1, 1, 1, validK>, Stride<validK, validK, validK, validK, 1>>;
    using GlobalB = GlobalTensor<BType, Shape<1, 1, 1, validK, validN>, Stride<validK * validN, validK * validN, validK * validN, validN, 1>>;
    using GlobalSA = GlobalTensor<ScaleType, Shape<1, 1, 1, 1, kMX>, Stride<kMX, kMX, kMX, kMX, 1>>;
    using GlobalSB = GlobalTensor<ScaleType, TileShape2D<ScaleType, kMX, validN, LB>, BaseShape2D<ScaleType, kMX, validN, LB>, LB>;
    using GlobalOut = GlobalTensor<float, Shape<1, 1, 1, 1, validN>, Stride<validN, validN, validN, validN, 1>>;
    GlobalA aGlobal(src0);
    GlobalB bGlobal(src1);
    GlobalSA saGlobal(src2);
    GlobalSB sbGlobal(src3);
    GlobalOut outGlobal(out);

    using MatA = Tile<TileType::Mat, AType, 1, KLeft, BLayout::RowMajor, 1, validK>;
    using MatSA = Tile<TileType::Mat, ScaleType, 1, kMX, BLayout::RowMajor, 1, kMX, SLayout::RowMajor, 32>;
    using MatB = Tile<TileType::Mat, BType, kAlign, N, BLayout::ColMajor, validK, validN, SLayout::RowMajor, 512>;
    using MatSB = Tile<TileType::Mat, ScaleType, kMX, N, BLayout::ColMajor, kMX, validN, SLayout::ColMajor, 32>;
    MatA aMat;
    MatB bMat;
    MatSA saMat;
    MatSB sbMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x1000);
    TASSIGN(saMat, 0x9000);
    TASSIGN(sbMat, 0xA000);

    TileLeft<AType, 1, KLeft, 1, validK> aTile;
    TileRightCompact<BType, kAlign, N, kAlign, validN> bTile;
    TileAccCompact<float, M, N, 1, validN> cTile;
    TileLeftScaleCompact<ScaleType, 1, kMX, 1, kMX> saTile;
    TileRightScaleCompact<ScaleType, kMX, N, kMX, validN> sbTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(saTile, GetScaleAddr(aTile.data()));
    TASSIGN(sbTile, GetScaleAddr(bTile.data()));
    TASSIGN(cTile, 0x0);

    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TFILLPAD(bMat, bMat);
    TLOAD<MatSA, GlobalSA>(saMat, saGlobal);
    TLOAD<MatSB, GlobalSB>(sbMat, sbGlobal);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);

    TEXTRACT(aTile, aMat, 0, 0);
    TEXTRACT(bTile, bMat, 0, 0);
    TMOV(saTile, saMat);
    TMOV(sbTile, sbMat);
    set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
    wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);

    TGEMV_MX(cTile, aTile, saTile, bTile, sbTile);
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    TSTORE(outGlobal, cTile);
}

// ---- TCVT on Vec tiles -----------------------------------------------------------------------------------------------
template <typename DstT, typename SrcT, int R, int C, int validC>
__global__ AICORE void RunTCVT(__gm__ DstT* dst, __gm__ SrcT* src, int mode, int sat)
{
    using SrcTile = Tile<TileType::Vec, SrcT, R, C, BLayout::RowMajor, R, validC>;
    using DstTile = Tile<TileType::Vec, DstT, R, C, BLayout::RowMajor, R, validC>;
    SrcTile srcTile;
    DstTile dstTile;
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, CeilAlign<int>(SrcTile::Bytes, 32));
    GlobalTensor<SrcT, Shape<1, 1, 1, R, validC>, Stride<R * validC, R * validC, R * validC, validC, 1>> srcGlobal(src);
    GlobalTensor<DstT, Shape<1, 1, 1, R, validC>, Stride<R * validC, R * validC, R * validC, validC, 1>> dstGlobal(dst);
    Event<Op::TLOAD, Op::TCVT> loaded = TLOAD(srcTile, srcGlobal);
    Event<Op::TCVT, Op::TSTORE_VEC> converted;
    if (sat < 0)
        converted = TCVT(dstTile, srcTile, static_cast<RoundMode>(mode), loaded);
    else
        converted = TCVT(dstTile, srcTile, static_cast<RoundMode>(mode), static_cast<SaturationMode>(sat), loaded);
    TSTORE(dstGlobal, dstTile, converted);
}

// ---- TFILLPAD ----------------------------------------------------------------------------------------------------------
// Vec form: dst takes src inside src's valid region and dst's pad value everywhere else; the whole R x C tile is stored
template <typename T, int R, int C, int validR, int validC, PadValue Pad>
__global__ AICORE void RunTFILLPAD_VEC(__gm__ T* dst, __gm__ T* src)
{
    using SrcTile = Tile<TileType::Vec, T, R, C, BLayout::RowMajor, validR, validC>;
    using DstTile = Tile<TileType::Vec, T, R, C, BLayout::RowMajor, R, C, SLayout::NoneBox, TileConfig::fractalABSize, Pad>;
    SrcTile srcTile;
    DstTile dstTile;
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, CeilAlign<int>(SrcTile::Bytes, 32));
    GlobalTensor<T, Shape<1, 1, 1, validR, validC>, Stride<validR * validC, validR * validC, validR * validC, validC, 1>> srcGlobal(src);
    GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>> dstGlobal(dst);
    TLOAD(srcTile, srcGlobal);
    TFILLPAD(dstTile, srcTile);
    TSTORE(dstGlobal, dstTile);
}
// Mat form, in place: the tile's storage is first filled with `junk` through a full-size alias, then the valid region is
// loaded and the rest cleared; the whole static extent is read back through the alias
template <typename T, int R, int C, int validR, int validC>
__global__ AICORE void RunTFILLPAD_MAT(__gm__ T* dst, __gm__ T* src, __gm__ T* junk)
{
    using Part = Tile<TileType::Mat, T, R, C, BLayout::ColMajor, validR, validC, SLayout::RowMajor, 512>;
    using Full = Tile<TileType::Mat, T, R, C, BLayout::ColMajor, R, C, SLayout::RowMajor, 512>;
    Part part;
    Full full;
    TASSIGN(part, 0x400);
    TASSIGN(full, 0x400);
    Tile<TileType::Vec, T, R, C, BLayout::RowMajor, R, C> vecTile;  // never TASSIGNed: starts at the base of UB
    GlobalTensor<T, Shape<1, 1, 1, validR, validC>, Stride<validR * validC, validR * validC, validR * validC, validC, 1>> srcGlobal(src);
    GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>> junkGlobal(junk), dstGlobal(dst);
    TLOAD(full, junkGlobal);
    TLOAD(part, srcGlobal);
    TFILLPAD(part, part);
    TMOV(vecTile, full);
    TSTORE(dstGlobal, vecTile);
}

// ---- TEXTRACT at nonzero offsets ---------------------------------------------------------------------------------------
// C = A[R0 : R0 + m, K0 : K0 + k] . B[K0 : K0 + k, C0 : C0 + n] cut out of larger Mat tiles
template <typename T, typename OutT, int MA, int KA, int NB, int m, int k, int n, int R0, int K0, int C0>
__global__ AICORE void RunTEXTRACT_SUB(__gm__ OutT* out, __gm__ T* a, __gm__ T* b)
{
    GlobalTensor<T, Shape<1, 1, 1, MA, KA>, Stride<MA * KA, MA * KA, MA * KA, KA, 1>> aGlobal(a);
    GlobalTensor<T, Shape<1, 1, 1, KA, NB>, Stride<KA * NB, KA * NB, KA * NB, NB, 1>> bGlobal(b);
    GlobalTensor<OutT, Shape<1, 1, 1, m, n>, Stride<m * n, m * n, m * n, n, 1>> outGlobal(out);
    Tile<TileType::Mat, T, MA, KA, BLayout::ColMajor, MA, KA, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, T, KA, NB, BLayout::ColMajor, KA, NB, SLayout::RowMajor, 512> bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, CeilAlign<int>(MA * KA * (int)sizeof(T), 512));
    TileLeft<T, m, k> aTile;
    TileRight<T, k, n> bTile;
    TileAcc<OutT, m, n> cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TEXTRACT(aTile, aMat, R0, K0);
    TEXTRACT(bTile, bMat, K0, C0);
    TMATMUL(cTile, aTile, bTile);
    TSTORE(outGlobal, cTile);
}

// ---- TSTORE<AtomicAdd>: every core adds its product onto what `out` already holds ---------------------------------------
template <typename OutT, typename T, int M, int K, int N>
__global__ AICORE void RunTSTORE_ATOMIC(__gm__ OutT* out, __gm__ T* a, __gm__ T* b)
{
    GlobalTensor<T, Shape<1, 1, 1, M, K>, Stride<M * K, M * K, M * K, K, 1>> aGlobal(a + (size_t)get_block_idx() * M * K);
    GlobalTensor<T, Shape<1, 1, 1, K, N>, Stride<K * N, K * N, K * N, N, 1>> bGlobal(b);
    using GlobalOut = GlobalTensor<OutT, Shape<1, 1, 1, M, N>, Stride<M * N, M * N, M * N, N, 1>>;
    GlobalOut outGlobal(out);
    constexpr int Mp = CeilAlign<int>(M, 16), Kp = CeilAlign<int>(K, sizeof(T) == 1 ? 32 : 16), Np = CeilAlign<int>(N, sizeof(T) == 1 ? 32 : 16);
    Tile<TileType::Mat, T, Mp, Kp, BLayout::ColMajor, M, K, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, T, Kp, Np, BLayout::ColMajor, K, N, SLayout::RowMajor, 512> bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x4000);
    TileLeft<T, Mp, Kp, M, K> aTile;
    TileRight<T, Kp, Np, K, N> bTile;
    using AccT = TileAcc<OutT, Mp, Np, M, N>;
    AccT cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMATMUL(cTile, aTile, bTile);
    TSTORE<AccT, GlobalOut, AtomicType::AtomicAdd>(outGlobal, cTile);
}

// ---- TMOV / TEXTRACT into an accumulator tile ---------------------------------------------------------------------------
// MODE 0: C0 [M][N] comes in through a Vec tile, TMOV places it in the accumulator, TMATMUL_ACC adds A B onto it.
// MODE 1: TEXTRACT<NormalRelu> takes the accumulator's start value from offset (8, 16) of a larger [M + 8][N + 16] Vec tile.
// MODE 2: accumulator to accumulator: C1 = A B, TMOV(C2, C1), C2 += A B.
template <typename OutT, typename T, int M, int K, int N, int MODE>
__global__ AICORE void RunTMOV_INTO_ACC(__gm__ OutT* out, __gm__ T* a, __gm__ T* b, __gm__ OutT* c0)
{
    GlobalTensor<T, Shape<1, 1, 1, M, K>, Stride<M * K, M * K, M * K, K, 1>> aGlobal(a);
    GlobalTensor<T, Shape<1, 1, 1, K, N>, Stride<K * N, K * N, K * N, N, 1>> bGlobal(b);
    GlobalTensor<OutT, Shape<1, 1, 1, M, N>, Stride<M * N, M * N, M * N, N, 1>> outGlobal(out);
    constexpr int Mp = CeilAlign<int>(M, 16), Kp = CeilAlign<int>(K, sizeof(T) == 1 ? 32 : 16), Np = CeilAlign<int>(N, sizeof(T) == 1 ? 32 : 16);
    Tile<TileType::Mat, T, Mp, Kp, BLayout::ColMajor, M, K, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, T, Kp, Np, BLayout::ColMajor, K, N, SLayout::RowMajor, 512> bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x4000);
    TileLeft<T, Mp, Kp, M, K> aTile;
    TileRight<T, Kp, Np, K, N> bTile;
    TileAcc<OutT, Mp, Np, M, N> cTile, c1Tile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(c1Tile, 0x4000);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    if constexpr (MODE == 0) {
        GlobalTensor<OutT, Shape<1, 1, 1, M, N>, Stride<M * N, M * N, M * N, N, 1>> c0Global(c0);
        Tile<TileType::Vec, OutT, Mp, Np, BLayout::RowMajor, M, N> c0Tile;
        TASSIGN(c0Tile, 0x0);
        TLOAD(c0Tile, c0Global);
        TMOV(cTile, c0Tile);
    } else if constexpr (MODE == 1) {
        constexpr int R = M + 8, C = N + 16, Rp = CeilAlign<int>(R, 16), Cp = CeilAlign<int>(C, 16);
        GlobalTensor<OutT, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>> c0Global(c0);
        Tile<TileType::Vec, OutT, Rp, Cp, BLayout::RowMajor, R, C> c0Tile;
        TASSIGN(c0Tile, 0x0);
        TLOAD(c0Tile, c0Global);
        TEXTRACT<decltype(cTile), decltype(c0Tile), ReluPreMode::NormalRelu>(cTile, c0Tile, 8, 16);
    } else {
        TMATMUL(c1Tile, aTile, bTile);
        TMOV(cTile, c1Tile);
    }
    TMATMUL_ACC(cTile, aTile, bTile);
    TSTORE(outGlobal, cTile);
}

// ---- 5-D global tensors: gather through TLOAD, scatter through TSTORE ----------------------------------------------------
// ND: Shape<2,3,4,8,16> with padded strides is a 192 x 16 logical matrix; DN: the same shape is 8 x 384.
// `packed` receives the logical matrix row-major; `scattered` (same 5-D geometry as the source) receives it back.
template <typename T, Layout L>
__global__ AICORE void RunGLOBAL_5D(__gm__ T* packed, __gm__ T* scattered, __gm__ T* src)
{
    constexpr bool nd = L == Layout::ND;
    constexpr int R = nd ? 2 * 3 * 4 * 8 : 8, C = nd ? 16 : 2 * 3 * 4 * 16;
    using S = Shape<2, 3, 4, 8, 16>;
    using St = std::conditional_t<nd, Stride<3 * 4 * 8 * 20 + 12, 4 * 8 * 20 + 4, 8 * 20, 20, 1>, Stride<3 * 4 * 16 * 10 + 6, 4 * 16 * 10 + 2, 16 * 10, 1, 10>>;
    GlobalTensor<T, S, St, L> srcGlobal(src), scatterGlobal(scattered);
    GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>> packedGlobal(packed);
    Tile<TileType::Vec, T, R, C, BLayout::RowMajor, R, C> tile;
    TASSIGN(tile, 0x0);
    TLOAD(tile, srcGlobal);
    TSTORE(packedGlobal, tile);
    TSTORE(scatterGlobal, tile);
}

// ---- fix-pipe forms of TMOV / TEXTRACT (accumulator -> Vec tile) ----------------------------------------------------------
// mode 0: TMOV with relu, f32 -> half        1: TMOV, scalar quant word -> int8        2: TMOV, per-column words -> half (relu)
// mode 3: TEXTRACT of the sub-block at (16, 32), scalar quant word -> int8             4: TEXTRACT (16, 32) plain f32 -> f32
template <typename VecT, typename AccElem, typename T, int M, int K, int N, int mode>
__global__ AICORE void RunTMOV_FIXPIPE(__gm__ VecT* out, __gm__ T* a, __gm__ T* b, __gm__ uint64_t* words)
{
    constexpr bool sub = mode >= 3;
    constexpr int VR = sub ? M - 16 : M, VC = sub ? N - 32 : N;
    GlobalTensor<T, Shape<1, 1, 1, M, K>, Stride<M * K, M * K, M * K, K, 1>> aGlobal(a);
    GlobalTensor<T, Shape<1, 1, 1, K, N>, Stride<K * N, K * N, K * N, N, 1>> bGlobal(b);
    GlobalTensor<VecT, Shape<1, 1, 1, VR, VC>, Stride<VR * VC, VR * VC, VR * VC, VC, 1>> outGlobal(out);
    GlobalTensor<uint64_t, Shape<1, 1, 1, 1, N>, Stride<N, N, N, N, 1>> wordsGlobal(words);
    Tile<TileType::Mat, T, M, K, BLayout::ColMajor, M, K, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, T, K, N, BLayout::ColMajor, K, N, SLayout::RowMajor, 512> bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x4000);
    TileLeft<T, M, K> aTile;
    TileRight<T, K, N> bTile;
    TileAcc<AccElem, M, N> cTile;
    Tile<TileType::Vec, VecT, VR, VC, BLayout::RowMajor, VR, VC> vTile;
    Tile<TileType::Scaling, uint64_t, 1, N, BLayout::RowMajor, 1, N> fpTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(vTile, 0x0);
    TASSIGN(fpTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMATMUL(cTile, aTile, bTile);
    TSYNC<Op::TMATMUL>();
    if constexpr (mode == 0) {
        TMOV<decltype(vTile), decltype(cTile), ReluPreMode::NormalRelu>(vTile, cTile);
    } else if constexpr (mode == 1) {
        TMOV(vTile, cTile, words[0]);
    } else if constexpr (mode == 2) {
        TLOAD(fpTile, wordsGlobal);
        TMOV<decltype(vTile), decltype(cTile), decltype(fpTile), ReluPreMode::NormalRelu>(vTile, cTile, fpTile);
    } else if constexpr (mode == 3) {
        TEXTRACT(vTile, cTile, words[0], (uint16_t)16, (uint16_t)32);
    } else {
        TEXTRACT(vTile, cTile, 16, 32);
    }
    TSTORE(outGlobal, vTile);
}

// ---- TRESHAPE: a 16 x 64 Vec tile seen as 8 x 128 over the same bytes ----------------------------------------------------
__global__ AICORE void RunTRESHAPE(__gm__ float* out, __gm__ float* src)
{
    Tile<TileType::Vec, float, 16, 64, BLayout::RowMajor, 16, 64> wide;
    Tile<TileType::Vec, float, 8, 128, BLayout::RowMajor, 8, 128> flat;
    TASSIGN(wide, 0x200);
    GlobalTensor<float, Shape<1, 1, 1, 16, 64>, Stride<1024, 1024, 1024, 64, 1>> srcGlobal(src);
    GlobalTensor<float, Shape<1, 1, 1, 8, 128>, Stride<1024, 1024, 1024, 128, 1>> outGlobal(out);
    TLOAD(wide, srcGlobal);
    TRESHAPE(flat, wide);
    TSTORE(outGlobal, flat);
}

// ---- TASSIGN outside the tile's region: the core carries on at offset 0 and the status word records it -----------------
__global__ AICORE void RunTASSIGN_OUT_OF_RANGE(__gm__ float* out, __gm__ float* src, uint32_t addr)
{
    Tile<TileType::Vec, float, 8, 32, BLayout::RowMajor, 8, 32> tile;
    TASSIGN(tile, addr);
    GlobalTensor<float, Shape<1, 1, 1, 8, 32>, Stride<256, 256, 256, 32, 1>> srcGlobal(src), outGlobal(out);
    TLOAD(tile, srcGlobal);
    TSTORE(outGlobal, tile);
}

// ---- launchers ---------------------------------------------------------------------------------------------------------
template <auto Kernel, typename... Args>
static int run(void* stream, int blocks, Args... args)
{
    return pto::amd::launch<Kernel>(blocks, stream, args...);
}

// block-scaled cases (shapes of tests/cpu/st/testcase/tmatmul_mx/main.cpp case2, 3, 5, 6, 15 and the two TGEMV_MX cases):
//   2: e4m3 x e4m3 127x72x64      3: e4m3 x e5m2 128x110x63     5: e1m2 x e2m1 117x64x60     6: e2m1 x e1m2 128x118x64
//   15: e2m1 x e1m2 35x128x56 + bias     11: gemv e1m2 x e1m2 1x128x62, B scales MX_B_ND     12: gemv e4m3 x e5m2 1x256x20, MX_B_ND
//   21: gemv e2m1 x e2m1 1x192x40, B scales MX_B_DN
// ---- quantise, then multiply: the step between TQUANT and TMATMUL_MX inside one kernel --------------------------------
// A arrives as f32.  TQUANT<MXFP8> turns it into E4M3 codes plus one E8M0 exponent per 32 elements in Vec (unified
// buffer) tiles; TMOV carries the codes from the row-major Vec tile into the fractal (NZ) Mat tile and the exponents,
// viewed as an [M][K/32] scale tile at the same unified-buffer address, into the scale Mat tile; from there on the
// kernel is the ordinary TMATMUL_MX pipeline.  B and its scales come quantised from global memory.
template <int M, int K, int N>
__global__ AICORE void RunQUANT_TMATMUL_MX(__gm__ float* out, __gm__ float* src0, __gm__ float8_e4m3_t* src1, __gm__ float8_e8m0_t* src3)
{
    using ScaleType = float8_e8m0_t;
    using E4 = float8_e4m3_t;
    constexpr int kMX = K / 32, G = M * kMX;
    static_assert(M % 16 == 0 && K % 64 == 0 && N % 32 == 0, "whole fractals");

    using SrcTile = Tile<TileType::Vec, float, M, K, BLayout::RowMajor, M, K>;
    using CodeTile = Tile<TileType::Vec, E4, M, K, BLayout::RowMajor, M, K>;
    using ExpTile = Tile<TileType::Vec, uint8_t, 1, G, BLayout::RowMajor, 1, G>;
    using ExpView = Tile<TileType::Vec, ScaleType, M, kMX, BLayout::RowMajor, M, kMX>;
    using FlatTile = Tile<TileType::Vec, float, 1, G, BLayout::RowMajor, 1, G>;
    SrcTile srcTile;
    CodeTile codeTile;
    ExpTile expTile;
    ExpView expView;
    FlatTile maxTile, scalingTile;
    constexpr int u1 = CeilAlign<int>(SrcTile::Bytes, 32), u2 = u1 + CeilAlign<int>(CodeTile::Bytes, 32),
                  u3 = u2 + CeilAlign<int>(ExpTile::Bytes, 32), u4 = u3 + CeilAlign<int>(FlatTile::Bytes, 32);
    TASSIGN(srcTile, 0x0);
    TASSIGN(codeTile, u1);
    TASSIGN(expTile, u2);
    TASSIGN(expView, u2);  // the same bytes, seen as M rows of K / 32 scales
    TASSIGN(maxTile, u3);
    TASSIGN(scalingTile, u4);

    using MatA = Tile<TileType::Mat, E4, M, K, BLayout::ColMajor, M, K, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, E4, K, N, BLayout::ColMajor, K, N, SLayout::RowMajor, 512>;
    using MatSA = Tile<TileType::Mat, ScaleType, M, kMX, BLayout::RowMajor, M, kMX, SLayout::RowMajor, 32>;
    using MatSB = Tile<TileType::Mat, ScaleType, kMX, N, BLayout::ColMajor, kMX, N, SLayout::ColMajor, 32>;
    MatA aMat;
    MatB bMat;
    MatSA saMat;
    MatSB sbMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, M * K);
    TASSIGN(saMat, M * K + K * N);
    TASSIGN(sbMat, M * K + K * N + M * kMX);
    TileLeft<E4, M, K, M, K> aTile;
    TileRight<E4, K, N, K, N> bTile;
    TileLeftScale<ScaleType, M, kMX, M, kMX> saTile;
    TileRightScale<ScaleType, kMX, N, kMX, N> sbTile;
    TileAcc<float, M, N, M, N> cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(saTile, GetScaleAddr(aTile.data()));
    TASSIGN(sbTile, GetScaleAddr(bTile.data()));

    GlobalTensor<float, TileShape2D<float, M, K>, BaseShape2D<float, M, K>> aGlobal(src0);
    GlobalTensor<E4, TileShape2D<E4, K, N>, BaseShape2D<E4, K, N>> bGlobal(src1);
    using GlobalSB = GlobalTensor<ScaleType, TileShape2D<ScaleType, kMX, N, Layout::MX_B_NN>, BaseShape2D<ScaleType, kMX, N, Layout::MX_B_NN>, Layout::MX_B_NN>;
    GlobalSB sbGlobal(src3);
    GlobalTensor<float, TileShape2D<float, M, N>, BaseShape2D<float, M, N>> outGlobal(out);

    TLOAD(srcTile, aGlobal);
    TLOAD(bMat, bGlobal);
    TLOAD<MatSB, GlobalSB>(sbMat, sbGlobal);
    set_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    TQUANT<QuantType::MXFP8>(codeTile, srcTile, &expTile, &maxTile, &scalingTile);
    set_flag(PIPE_V, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_V, PIPE_MTE1, EVENT_ID0);
    TMOV(aMat, codeTile);   // codes: ND (row-major Vec tile) -> NZ (fractal Mat tile)
    TMOV(saMat, expView);   // exponents: [M][K / 32] rows -> the scale Mat tile
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMOV(saTile, saMat);
    TMOV(sbTile, sbMat);
    set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
    wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
    TMATMUL_MX(cTile, aTile, saTile, bTile, sbTile);
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    TSTORE(outGlobal, cTile);
}

// Packed fp4 operands from either global layout, through the element-wise TLOAD (the tiles are not fully valid, so the
// LDS-DMA form does not apply): A as ND (codes paired along a row, as the row-lined Mat tile pairs them) or DN (paired
// down a column: every tile byte is built from two bytes of memory); B as DN (paired down a column, as the column-lined
// Mat tile pairs them) or ND.  The Left / Right tiles are copies (zero-filled past the valid region).
template <bool A_DN, bool B_DN, int validM, int validK, int validN>
__global__ AICORE void RunTMATMULMX_FP4_LAYOUTS(__gm__ float* out, __gm__ float4_e2m1x2_t* src0, __gm__ float4_e2m1x2_t* src1,
                                                __gm__ float8_e8m0_t* src2, __gm__ float8_e8m0_t* src3)
{
    using F4 = float4_e2m1x2_t;
    using X = float8_e8m0_t;
    constexpr int M = CeilAlign<int>(validM, 32), N = CeilAlign<int>(validN, 32), K = CeilAlign<int>(validK, 64), kMX = K / 32;
    constexpr Layout LA = A_DN ? Layout::DN : Layout::ND, LB = B_DN ? Layout::DN : Layout::ND;
    GlobalTensor<F4, TileShape2D<F4, validM, validK, LA>, BaseShape2D<F4, validM, validK, LA>, LA> aGlobal(src0);
    GlobalTensor<F4, TileShape2D<F4, validK, validN, LB>, BaseShape2D<F4, validK, validN, LB>, LB> bGlobal(src1);
    GlobalTensor<X, TileShape2D<X, validM, validK / 32, Layout::MX_A_ND>, BaseShape2D<X, validM, validK / 32, Layout::MX_A_ND>, Layout::MX_A_ND>
        saGlobal(src2);
    GlobalTensor<X, TileShape2D<X, validK / 32, validN, Layout::MX_B_DN>, BaseShape2D<X, validK / 32, validN, Layout::MX_B_DN>, Layout::MX_B_DN>
        sbGlobal(src3);
    GlobalTensor<float, TileShape2D<float, validM, validN>, BaseShape2D<float, validM, validN>> outGlobal(out);
    Tile<TileType::Mat, F4, M, K, BLayout::ColMajor, validM, validK, SLayout::RowMajor> aMat;
    Tile<TileType::Mat, F4, K, N, BLayout::RowMajor, validK, validN, SLayout::ColMajor> bMat;
    Tile<TileType::Mat, X, M, kMX, BLayout::RowMajor, validM, validK / 32, SLayout::RowMajor, 32> saMat;
    Tile<TileType::Mat, X, kMX, N, BLayout::ColMajor, validK / 32, validN, SLayout::ColMajor, 32> sbMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, M * K / 2);
    TASSIGN(saMat, M * K / 2 + K * N / 2);
    TASSIGN(sbMat, M * K / 2 + K * N / 2 + M * kMX);
    TileLeft<F4, M, K, validM, validK> aTile;
    TileRight<F4, K, N, validK, validN> bTile;
    TileLeftScale<X, M, kMX, validM, validK / 32> saTile;
    TileRightScale<X, kMX, N, validK / 32, validN> sbTile;
    TileAcc<float, M, N, validM, validN> cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(saTile, 0x0);
    TASSIGN(sbTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TLOAD(saMat, saGlobal);
    TLOAD(sbMat, sbGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMOV(saTile, saMat);
    TMOV(sbTile, sbMat);
    TMATMUL_MX(cTile, aTile, saTile, bTile, sbTile);
    TSTORE(outGlobal, cTile);
}

extern "C" int pto_boundary_launch_mx(int id, void* out, void* a, void* b, void* sa, void* sb, void* bias, void* stream)
{
    using S = float8_e8m0_t;
    using E4 = float8_e4m3_t;
    using E5 = float8_e5m2_t;
    using F21 = float4_e2m1x2_t;
    using F12 = float4_e1m2x2_t;
    switch (id) {
    case 2: return run<&RunTMATMULMX<E4, E4, 127, 72, 64, false, false>>(stream, 1, (float*)out, (E4*)a, (E4*)b, (S*)sa, (S*)sb, (float*)bias);
    case 3: return run<&RunTMATMULMX<E4, E5, 128, 110, 63, false, false>>(stream, 1, (float*)out, (E4*)a, (E5*)b, (S*)sa, (S*)sb, (float*)bias);
    case 5: return run<&RunTMATMULMX<F12, F21, 117, 64, 60, false, true>>(stream, 1, (float*)out, (F12*)a, (F21*)b, (S*)sa, (S*)sb, (float*)bias);
    case 6: return run<&RunTMATMULMX<F21, F12, 128, 118, 64, false, true>>(stream, 1, (float*)out, (F21*)a, (F12*)b, (S*)sa, (S*)sb, (float*)bias);
    case 15: return run<&RunTMATMULMX<F21, F12, 35, 128, 56, true, true>>(stream, 1, (float*)out, (F21*)a, (F12*)b, (S*)sa, (S*)sb, (float*)bias);
    case 11: return run<&RunTGEMVMX<F12, F12, 128, 62, Layout::MX_B_ND, true>>(stream, 1, (float*)out, (F12*)a, (F12*)b, (S*)sa, (S*)sb);
    case 12: return run<&RunTGEMVMX<E4, E5, 256, 20, Layout::MX_B_ND, false>>(stream, 1, (float*)out, (E4*)a, (E5*)b, (S*)sa, (S*)sb);
    case 21: return run<&RunTGEMVMX<F21, F21, 192, 40, Layout::MX_B_DN, true>>(stream, 1, (float*)out, (F21*)a, (F21*)b, (S*)sa, (S*)sb);
    // 30-33: fp4 operands from ND / DN global tensors (30 + (A is DN) + 2 (B is DN)), 30 x 128 x 60 valid
    case 30: return run<&RunTMATMULMX_FP4_LAYOUTS<false, false, 30, 128, 60>>(stream, 1, (float*)out, (F21*)a, (F21*)b, (S*)sa, (S*)sb);
    case 31: return run<&RunTMATMULMX_FP4_LAYOUTS<true, false, 30, 128, 60>>(stream, 1, (float*)out, (F21*)a, (F21*)b, (S*)sa, (S*)sb);
    case 32: return run<&RunTMATMULMX_FP4_LAYOUTS<false, true, 30, 128, 60>>(stream, 1, (float*)out, (F21*)a, (F21*)b, (S*)sa, (S*)sb);
    case 33: return run<&RunTMATMULMX_FP4_LAYOUTS<true, true, 30, 128, 60>>(stream, 1, (float*)out, (F21*)a, (F21*)b, (S*)sa, (S*)sb);
    default: return -1;
    }
}

// TCVT cases, 16 x 72 tiles with 70 valid columns:
//   1: f32 -> half     2: f32 -> bf16     3: f32 -> int32     4: f32 -> int8     5: f32 -> uint8     6: f32 -> e4m3
//   7: f32 -> e5m2     8: half -> f32     9: int32 -> f32     10: half -> int16   11: e4m3 -> f32    12: half -> e4m3
// sat < 0 calls the overload without a saturation mode
extern "C" int pto_boundary_launch_cvt(int id, void* dst, void* src, int mode, int sat, void* stream)
{
    constexpr int R = 16, C = 72, V = 70;
    switch (id) {
    case 1: return run<&RunTCVT<half, float, R, C, V>>(stream, 1, (half*)dst, (float*)src, mode, sat);
    case 2: return run<&RunTCVT<bfloat16_t, float, R, C, V>>(stream, 1, (bfloat16_t*)dst, (float*)src, mode, sat);
    case 3: return run<&RunTCVT<int32_t, float, R, C, V>>(stream, 1, (int32_t*)dst, (float*)src, mode, sat);
    case 4: return run<&RunTCVT<int8_t, float, R, C, V>>(stream, 1, (int8_t*)dst, (float*)src, mode, sat);
    case 5: return run<&RunTCVT<uint8_t, float, R, C, V>>(stream, 1, (uint8_t*)dst, (float*)src, mode, sat);
    case 6: return run<&RunTCVT<float8_e4m3_t, float, R, C, V>>(stream, 1, (float8_e4m3_t*)dst, (float*)src, mode, sat);
    case 7: return run<&RunTCVT<float8_e5m2_t, float, R, C, V>>(stream, 1, (float8_e5m2_t*)dst, (float*)src, mode, sat);
    case 8: return run<&RunTCVT<float, half, R, C, V>>(stream, 1, (float*)dst, (half*)src, mode, sat);
    case 9: return run<&RunTCVT<float, int32_t, R, C, V>>(stream, 1, (float*)dst, (int32_t*)src, mode, sat);
    case 10: return run<&RunTCVT<int16_t, half, R, C, V>>(stream, 1, (int16_t*)dst, (half*)src, mode, sat);
    case 11: return run<&RunTCVT<float, float8_e4m3_t, R, C, V>>(stream, 1, (float*)dst, (float8_e4m3_t*)src, mode, sat);
    case 12: return run<&RunTCVT<float8_e4m3_t, half, R, C, V>>(stream, 1, (float8_e4m3_t*)dst, (half*)src, mode, sat);
    default: return -1;
    }
}

// other cases:
//   1: TFILLPAD Vec f32 16x64 valid 13x50 pad Max     2: same, pad Min, half     3: same, pad Zero, int32
//   4: TFILLPAD Mat in place, half 32x64 valid 27x40   5: same, e4m3 32x64 valid 32x33
//   10: TEXTRACT sub-blocks half: A 64x128, B 128x64 -> A[32:64, 64:128] . B[64:128, 32:64]
//   11: TEXTRACT sub-blocks int8: A 32x128, B 128x64 -> A[16:32, 32:96] . B[32:96, 32:64]
//   20: TSTORE<AtomicAdd> f32 40x50x60, 3 cores (a holds 3 A matrices)     21: int32 from int8 24x64x40, 2 cores
//   30 / 31: 5-D global tensor half ND / DN (out = packed, src1 = scattered)     32: float ND
//   40..44: fix-pipe TMOV / TEXTRACT modes 0..4 on a half 48x64x96 product (src2 = quant words)
//   45: mode 1 on an int8 48x64x96 product (int32 accumulator -> int8)
//   46-49: TMOV / TEXTRACT into an accumulator tile (from a Vec tile, with relu at an offset, from another accumulator; int32)
//   50: TRESHAPE     60: TASSIGN at the address in `arg`     70: TQUANT<MXFP8> of an f32 A, TMOV ND -> NZ, TMATMUL_MX
extern "C" int pto_boundary_launch(int id, void* out, void* src0, void* src1, void* src2, unsigned arg, void* stream)
{
    using E4 = float8_e4m3_t;
    switch (id) {
    case 1: return run<&RunTFILLPAD_VEC<float, 16, 64, 13, 50, PadValue::Max>>(stream, 1, (float*)out, (float*)src0);
    case 2: return run<&RunTFILLPAD_VEC<half, 16, 64, 13, 50, PadValue::Min>>(stream, 1, (half*)out, (half*)src0);
    case 3: return run<&RunTFILLPAD_VEC<int32_t, 16, 64, 13, 50, PadValue::Zero>>(stream, 1, (int32_t*)out, (int32_t*)src0);
    case 4: return run<&RunTFILLPAD_MAT<half, 32, 64, 27, 40>>(stream, 1, (half*)out, (half*)src0, (half*)src1);
    case 5: return run<&RunTFILLPAD_MAT<E4, 32, 64, 32, 33>>(stream, 1, (E4*)out, (E4*)src0, (E4*)src1);
    case 10: return run<&RunTEXTRACT_SUB<half, float, 64, 128, 64, 32, 64, 32, 32, 64, 32>>(stream, 1, (float*)out, (half*)src0, (half*)src1);
    case 11: return run<&RunTEXTRACT_SUB<int8_t, int32_t, 32, 128, 64, 16, 64, 32, 16, 32, 32>>(stream, 1, (int32_t*)out, (int8_t*)src0, (int8_t*)src1);
    case 20: return run<&RunTSTORE_ATOMIC<float, half, 40, 50, 60>>(stream, 3, (float*)out, (half*)src0, (half*)src1);
    case 21: return run<&RunTSTORE_ATOMIC<int32_t, int8_t, 24, 64, 40>>(stream, 2, (int32_t*)out, (int8_t*)src0, (int8_t*)src1);
    case 30: return run<&RunGLOBAL_5D<half, Layout::ND>>(stream, 1, (half*)out, (half*)src1, (half*)src0);
    case 31: return run<&RunGLOBAL_5D<half, Layout::DN>>(stream, 1, (half*)out, (half*)src1, (half*)src0);
    case 32: return run<&RunGLOBAL_5D<float, Layout::ND>>(stream, 1, (float*)out, (float*)src1, (float*)src0);
    case 40: return run<&RunTMOV_FIXPIPE<half, float, half, 48, 64, 96, 0>>(stream, 1, (half*)out, (half*)src0, (half*)src1, (uint64_t*)src2);
    case 41: return run<&RunTMOV_FIXPIPE<int8_t, float, half, 48, 64, 96, 1>>(stream, 1, (int8_t*)out, (half*)src0, (half*)src1, (uint64_t*)src2);
    case 42: return run<&RunTMOV_FIXPIPE<half, float, half, 48, 64, 96, 2>>(stream, 1, (half*)out, (half*)src0, (half*)src1, (uint64_t*)src2);
    case 43: return run<&RunTMOV_FIXPIPE<int8_t, float, half, 48, 64, 96, 3>>(stream, 1, (int8_t*)out, (half*)src0, (half*)src1, (uint64_t*)src2);
    case 44: return run<&RunTMOV_FIXPIPE<float, float, half, 48, 64, 96, 4>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (uint64_t*)src2);
    case 45: return run<&RunTMOV_FIXPIPE<int8_t, int32_t, int8_t, 48, 64, 96, 1>>(stream, 1, (int8_t*)out, (int8_t*)src0, (int8_t*)src1, (uint64_t*)src2);
    case 46: return run<&RunTMOV_INTO_ACC<float, half, 40, 50, 60, 0>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)src2);
    case 47: return run<&RunTMOV_INTO_ACC<float, half, 40, 50, 60, 1>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)src2);
    case 48: return run<&RunTMOV_INTO_ACC<float, half, 40, 50, 60, 2>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)src2);
    case 49: return run<&RunTMOV_INTO_ACC<int32_t, int8_t, 24, 64, 40, 0>>(stream, 1, (int32_t*)out, (int8_t*)src0, (int8_t*)src1, (int32_t*)src2);
    case 50: return run<&RunTRESHAPE>(stream, 1, (float*)out, (float*)src0);
    case 60: return run<&RunTASSIGN_OUT_OF_RANGE>(stream, 1, (float*)out, (float*)src0, (uint32_t)arg);
    case 70: return run<&RunQUANT_TMATMUL_MX<32, 128, 64>>(stream, 1, (float*)out, (float*)src0, (E4*)src1, (float8_e8m0_t*)src2);
    default: return -1;
    }
}

extern "C" int pto_boundary_status() { return pto::amd::device_status(); }
extern "C" int pto_boundary_reset_status() { return pto::amd::reset_device_status(); }
