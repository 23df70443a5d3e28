// PTO-style kernel sources for the gfx950 backend, written against <pto/pto-inst.hpp> the way the reference's own test
// kernels are (tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:25-173 is the model for the single-tile and split-K
// programs, demos/cpu/gemm_demo/gemm_demo.cpp:83-121 for the tiled GEMM), plus the extern "C" launchers the parity
// tests call.  Inputs and outputs are device pointers.
#include <pto/pto-inst.hpp>
#include <pto/common/constants.hpp>

using namespace pto;

template <typename T>
AICORE constexpr inline T CeilAlign(T a, T b)
{
    return b == 0 ? 0 : (a + b - 1) / b * b;
}

// One tile: C[validM, validN] = A[validM, validK] . B[validK, validN] (+ bias), all row-major in global memory.
template <typename OutT, typename AT, typename BT, typename BiasT, int validM, int validK, int validN, bool isBias>
__global__ AICORE void RunTMATMUL(__gm__ OutT* out, __gm__ AT* src0, __gm__ BT* src1, __gm__ BiasT* src2)
{
    constexpr int blockAlign = (sizeof(AT) == 1) ? 32 : 16;
    constexpr int M = CeilAlign<int>(validM, 16);
    constexpr int N = CeilAlign<int>(validN, blockAlign);
    constexpr int K = CeilAlign<int>(validK, blockAlign);

    using GlobalA = GlobalTensor<AT, Shape<1, 1, 1, validM, validK>, Stride<validM * validK, validM * validK, validM * validK, validK, 1>>;
    using GlobalB = GlobalTensor<BT, Shape<1, 1, 1, validK, validN>, Stride<validK * validN, validK * validN, validK * validN, validN, 1>>;
    using GlobalBias = GlobalTensor<BiasT, Shape<1, 1, 1, 1, validN>, Stride<validN, validN, validN, validN, 1>>;
    using GlobalOut = GlobalTensor<OutT, Shape<1, 1, 1, validM, validN>, Stride<validM * validN, validM * validN, validM * validN, validN, 1>>;
    GlobalA aGlobal(src0);
    GlobalB bGlobal(src1);
    GlobalOut outGlobal(out);

    using MatA = Tile<TileType::Mat, AT, M, K, BLayout::ColMajor, validM, validK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, BT, K, N, BLayout::ColMajor, validK, validN, SLayout::RowMajor, 512>;
    using LeftT = TileLeft<AT, M, K, validM, validK>;
    using RightT = TileRight<BT, K, N, validK, validN>;
    using AccT = TileAcc<OutT, M, N, validM, validN>;
    using BiasTile = Tile<TileType::Bias, BiasT, 1, N, BLayout::RowMajor, 1, validN>;

    MatA aMat;
    MatB bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    LeftT aTile;
    RightT bTile;
    AccT cTile;
    BiasTile biasTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(biasTile, 0x0);

    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);

    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
    wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);

    if constexpr (isBias) {
        GlobalBias biasGlobal(src2);
        TLOAD(biasTile, biasGlobal);
        if constexpr (validM == 1)
            TGEMV_BIAS(cTile, aTile, bTile, biasTile);
        else
            TMATMUL_BIAS(cTile, aTile, bTile, biasTile);
    } else {
        if constexpr (validM == 1)
            TGEMV(cTile, aTile, bTile);
        else
            TMATMUL(cTile, aTile, bTile);
    }
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    TSTORE(outGlobal, cTile);
}

// numRepeats K-slabs accumulated into one accumulator tile: TMATMUL for the first, TMATMUL_ACC after
template <typename OutT, typename AT, typename BT, int M, int K, int N>
__global__ AICORE void RunTMATMUL_SPLIT_K(__gm__ OutT* out, __gm__ AT* src0, __gm__ BT* src1, uint32_t numRepeats)
{
    using GlobalA = GlobalTensor<AT, Shape<1, 1, 1, M, K>, Stride<M * K, M * K, M * K, K, 1>>;
    using GlobalB = GlobalTensor<BT, Shape<1, 1, 1, K, N>, Stride<K * N, K * N, K * N, N, 1>>;
    using GlobalOut = GlobalTensor<OutT, Shape<1, 1, 1, M, N>, Stride<M * N, M * N, M * N, N, 1>>;
    GlobalOut outGlobal(out);
    using MatA = Tile<TileType::Mat, AT, M, K, BLayout::ColMajor, M, K, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, BT, K, N, BLayout::ColMajor, K, N, SLayout::RowMajor, 512>;
    MatA aMat;
    MatB bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    TileLeft<AT, M, K> aTile;
    TileRight<BT, K, N> bTile;
    TileAcc<OutT, M, N> cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    for (uint32_t i = 0; i < numRepeats; i++) {
        GlobalA aGlobal(src0 + i * M * K);
        GlobalB bGlobal(src1 + i * K * N);
        TLOAD(aMat, aGlobal);
        TLOAD(bMat, bGlobal);
        TMOV(aTile, aMat);
        TMOV(bTile, bMat);
        if (i == 0)
            TMATMUL(cTile, aTile, bTile);
        else
            TMATMUL_ACC(cTile, cTile, aTile, bTile);
    }
    TSTORE(outGlobal, cTile);
}

// Block-scaled single tile: C = sum_k A(i, k) B(k, j) 2^(sa(i, k/32) - 127) 2^(sb(k/32, j) - 127) (+ bias).  A is [M][K],
// B is [K][N] row-major, one byte per element; the E8M0 scales sit in global memory in the layouts named by LA / LB
// (logical [M][K/32] and [K/32][N]).  Structure after tests/cpu/st/testcase/tmatmul_mx/tmatmul_mx_kernel.cpp:66-200.
template <typename AT, typename BT, int validM, int validK, int validN, Layout LA, Layout LB, bool isBias>
__global__ AICORE void RunTMATMUL_MX(__gm__ float* out, __gm__ AT* src0, __gm__ BT* src1, __gm__ float8_e8m0_t* src2,
                                     __gm__ float8_e8m0_t* src3, __gm__ float* src4)
{
    using ScaleType = float8_e8m0_t;
    constexpr int M = CeilAlign<int>(validM, 16), N = CeilAlign<int>(validN, 32), K = CeilAlign<int>(validK, 64);
    constexpr int kMX = K / 32, validKMX = validK / 32;
    static_assert(validK % 64 == 0, "MX matmul needs K to be a multiple of 64");

    using GlobalA = GlobalTensor<AT, TileShape2D<AT, validM, validK>, BaseShape2D<AT, validM, validK>>;
    using GlobalB = GlobalTensor<BT, TileShape2D<BT, validK, validN>, BaseShape2D<BT, validK, validN>>;
    using GlobalSA = GlobalTensor<ScaleType, TileShape2D<ScaleType, validM, validKMX, LA>, BaseShape2D<ScaleType, validM, validKMX, LA>, LA>;
    using GlobalSB = GlobalTensor<ScaleType, TileShape2D<ScaleType, validKMX, validN, LB>, BaseShape2D<ScaleType, validKMX, validN, LB>, LB>;
    using GlobalBias = GlobalTensor<float, TileShape2D<float, 1, validN>, BaseShape2D<float, 1, validN>>;
    using GlobalOut = GlobalTensor<float, TileShape2D<float, validM, validN>, BaseShape2D<float, validM, validN>>;
    GlobalA aGlobal(src0);
    GlobalB bGlobal(src1);
    GlobalSA saGlobal(src2);
    GlobalSB sbGlobal(src3);
    GlobalOut outGlobal(out);

    using MatA = Tile<TileType::Mat, AT, M, K, BLayout::ColMajor, validM, validK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, BT, K, N, BLayout::ColMajor, validK, validN, SLayout::RowMajor, 512>;
    using MatSA = Tile<TileType::Mat, ScaleType, M, kMX, BLayout::RowMajor, validM, validKMX, SLayout::RowMajor, 32>;
    using MatSB = Tile<TileType::Mat, ScaleType, kMX, N, BLayout::ColMajor, validKMX, validN, SLayout::ColMajor, 32>;
    using BiasMat = Tile<TileType::Mat, float, 1, N, BLayout::RowMajor, 1, validN>;
    MatA aMat;
    MatB bMat;
    MatSA saMat;
    MatSB sbMat;
    BiasMat biasMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, M * K);
    TASSIGN(saMat, M * K + K * N);
    TASSIGN(sbMat, M * K + K * N + M * kMX);
    TASSIGN(biasMat, M * K + K * N + M * kMX + N * kMX);

    TileLeft<AT, M, K, validM, validK> aTile;
    TileRight<BT, K, N, validK, validN> bTile;
    TileLeftScale<ScaleType, M, kMX, validM, validKMX> saTile;
    TileRightScale<ScaleType, kMX, N, validKMX, validN> sbTile;
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
    TLOAD<MatSA, GlobalSA>(saMat, saGlobal);
    TLOAD<MatSB, GlobalSB>(sbMat, sbGlobal);
    if constexpr (isBias) {
        GlobalBias biasGlobal(src4);
        TLOAD(biasMat, biasGlobal);
    }
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

// A in the NZ global layout (column blocks of 16 halves, rows contiguous inside a block), result moved Acc -> Vec tile
// (converted to half) and stored from there
template <int M, int K, int N>
__global__ AICORE void RunTMATMUL_NZ_VEC(__gm__ half* out, __gm__ half* src0, __gm__ half* src1)
{
    GlobalTensor<half, TileShape2D<half, M, K, Layout::NZ>, BaseShape2D<half, M, K, Layout::NZ>, Layout::NZ> aGlobal(src0);
    GlobalTensor<half, TileShape2D<half, K, N>, BaseShape2D<half, K, N>> bGlobal(src1);
    GlobalTensor<half, TileShape2D<half, M, N>, BaseShape2D<half, M, N>> outGlobal(out);
    Tile<TileType::Mat, half, M, K, BLayout::ColMajor, M, K, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, half, K, N, BLayout::ColMajor, K, N, SLayout::RowMajor, 512> bMat;
    TileLeft<half, M, K> aTile;
    TileRight<half, K, N> bTile;
    TileAcc<float, M, N> cTile;
    Tile<TileType::Vec, half, M, N, BLayout::RowMajor, M, N> vTile;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(vTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMATMUL(cTile, aTile, bTile);
    TMOV(vTile, cTile);
    TSTORE(outGlobal, vTile);
}

// The tiled GEMM of the CPU-simulator demo at full problem size: C[M, N] = A[M, K] . B[K, N], one core per BM x BN
// output tile, K walked in BK slabs through TLOAD -> TMOV -> TMATMUL / TMATMUL_ACC, then TSTORE of the tile.
template <typename OutT, typename InT, int M, int K, int N, int BM, int BN, int BK, bool B_IS_DN>
__global__ AICORE void RunTiledGemm(__gm__ OutT* out, __gm__ InT* a, __gm__ InT* b)
{
    constexpr int tilesN = N / BN;
    const int tile = (int)get_block_idx();
    const int tm = tile / tilesN, tn = tile % tilesN;

    using GlobalA = GlobalTensor<InT, Shape<1, 1, 1, BM, BK>, Stride<M * K, M * K, M * K, K, 1>>;
    // B is [K][N] row-major (ND view) or [N][K] in memory (the DN view of the same logical K x N matrix)
    using GlobalB = std::conditional_t<B_IS_DN, GlobalTensor<InT, Shape<1, 1, 1, BK, BN>, Stride<K * N, K * N, K * N, 1, K>, Layout::DN>,
                                       GlobalTensor<InT, Shape<1, 1, 1, BK, BN>, Stride<K * N, K * N, K * N, N, 1>>>;
    using GlobalOut = GlobalTensor<OutT, Shape<1, 1, 1, BM, BN>, Stride<M * N, M * N, M * N, N, 1>>;

    using MatA = Tile<TileType::Mat, InT, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, InT, BK, BN, BLayout::ColMajor, BK, BN, SLayout::RowMajor, 512>;
    MatA aMat;
    MatB bMat;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    TileLeft<InT, BM, BK> aTile;
    TileRight<InT, BK, BN> bTile;
    TileAcc<float, BM, BN> cTile;
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);

    for (int k0 = 0; k0 < K; k0 += BK) {
        GlobalA aGlobal(a + (size_t)tm * BM * K + k0);
        GlobalB bGlobal(B_IS_DN ? b + (size_t)tn * BN * K + k0 : b + (size_t)k0 * N + tn * BN);
        TLOAD(aMat, aGlobal);
        TLOAD(bMat, bGlobal);
        TMOV(aTile, aMat);
        TMOV(bTile, bMat);
        if (k0 == 0)
            TMATMUL(cTile, aTile, bTile);
        else
            TMATMUL_ACC(cTile, cTile, aTile, bTile);
    }
    GlobalOut outGlobal(out + (size_t)tm * BM * N + tn * BN);
    TSTORE(outGlobal, cTile);
}

// ---- launchers ------------------------------------------------------------------------------------------------------
// case ids follow the reference's tmatmul test list (tests/cpu/st/testcase/tmatmul/main.cpp:96-252):
//   1: f16 40x50x60 -> f32      2: int8 6x7x8 -> i32        3: f16 128x128x64, 5 K-slabs (split-K) -> f32
//   4: f32 56x110x40 -> f32     5: f16 gemv 1x110x50        6: f32 gemv 1x128x48       7: bf16 40x50x60 -> f32
//   8: fp8 e4m3 33x64x70 -> f32 (f32 shapes are smaller than the reference's: three copies of a tile - L1, L0 and
//   the accumulator - share 160 KiB of LDS here, not 512 + 64 + 64 KiB)
//   11: f16 + f32 bias 26x100x94          12: int8 + i32 bias 8x7x6 ... (bias cases)
//   100: tiled f16 512^3 -> f32 (B row-major)   101: tiled bf16 512x512x512 -> bf16 out (B column-major)
template <auto Kernel, typename... Args>
static int run(void* stream, int blocks, Args... args)
{
    return pto::amd::launch<Kernel>(blocks, stream, args...);
}

extern "C" int pto_kernels_launch(int id, void* out, void* src0, void* src1, void* src2, void* stream)
{
    switch (id) {
    case 1: return run<&RunTMATMUL<float, half, half, float, 40, 50, 60, false>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)nullptr);
    case 2: return run<&RunTMATMUL<int32_t, int8_t, int8_t, int32_t, 6, 7, 8, false>>(stream, 1, (int32_t*)out, (int8_t*)src0, (int8_t*)src1, (int32_t*)nullptr);
    case 3: return run<&RunTMATMUL_SPLIT_K<float, half, half, 128, 128, 64>>(stream, 1, (float*)out, (half*)src0, (half*)src1, 5u);
    case 4: return run<&RunTMATMUL<float, float, float, float, 56, 110, 40, false>>(stream, 1, (float*)out, (float*)src0, (float*)src1, (float*)nullptr);
    case 5: return run<&RunTMATMUL<float, half, half, float, 1, 110, 50, false>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)nullptr);
    case 6: return run<&RunTMATMUL<float, float, float, float, 1, 128, 48, false>>(stream, 1, (float*)out, (float*)src0, (float*)src1, (float*)nullptr);
    case 7: return run<&RunTMATMUL<float, bfloat16_t, bfloat16_t, float, 40, 50, 60, false>>(stream, 1, (float*)out, (bfloat16_t*)src0, (bfloat16_t*)src1, (float*)nullptr);
    case 8: return run<&RunTMATMUL<float, float8_e4m3_t, float8_e4m3_t, float, 33, 64, 70, false>>(stream, 1, (float*)out, (float8_e4m3_t*)src0, (float8_e4m3_t*)src1, (float*)nullptr);
    case 11: return run<&RunTMATMUL<float, half, half, float, 26, 100, 94, true>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)src2);
    case 12: return run<&RunTMATMUL<int32_t, int8_t, int8_t, int32_t, 8, 7, 6, true>>(stream, 1, (int32_t*)out, (int8_t*)src0, (int8_t*)src1, (int32_t*)src2);
    case 13: return run<&RunTMATMUL<float, half, half, float, 1, 64, 96, true>>(stream, 1, (float*)out, (half*)src0, (half*)src1, (float*)src2);
    case 20: return run<&RunTMATMUL_NZ_VEC<32, 64, 48>>(stream, 1, (half*)out, (half*)src0, (half*)src1);
    case 100: return run<&RunTiledGemm<float, half, 512, 512, 512, 128, 128, 64, false>>(stream, 16, (float*)out, (half*)src0, (half*)src1);
    case 101: return run<&RunTiledGemm<bfloat16_t, bfloat16_t, 512, 512, 512, 128, 128, 64, true>>(stream, 16, (bfloat16_t*)out, (bfloat16_t*)src0, (bfloat16_t*)src1);
    default: return -1;
    }
}

// MX cases: 1: e4m3 x e4m3 32x128x48, scales MX_A_ZZ / MX_B_NN      2: e5m2 x e4m3 33x192x70, scales MX_A_ND / MX_B_DN, bias
//           3: e4m3 x e5m2 16x64x32, scales MX_A_DN / MX_B_ND      4: e2m1 x e2m1 (packed fp4) 40x128x60, ND / DN scales
//           5: e2m1 x e2m1 32x256x64, scales MX_A_ZZ / MX_B_NN, bias
extern "C" int pto_kernels_launch_mx(int id, void* out, void* a, void* b, void* sa, void* sb, void* bias, void* stream)
{
    using S = float8_e8m0_t;
    switch (id) {
    case 1: return run<&RunTMATMUL_MX<float8_e4m3_t, float8_e4m3_t, 32, 128, 48, Layout::MX_A_ZZ, Layout::MX_B_NN, false>>(
            stream, 1, (float*)out, (float8_e4m3_t*)a, (float8_e4m3_t*)b, (S*)sa, (S*)sb, (float*)nullptr);
    case 2: return run<&RunTMATMUL_MX<float8_e5m2_t, float8_e4m3_t, 33, 192, 70, Layout::MX_A_ND, Layout::MX_B_DN, true>>(
            stream, 1, (float*)out, (float8_e5m2_t*)a, (float8_e4m3_t*)b, (S*)sa, (S*)sb, (float*)bias);
    case 3: return run<&RunTMATMUL_MX<float8_e4m3_t, float8_e5m2_t, 16, 64, 32, Layout::MX_A_DN, Layout::MX_B_ND, false>>(
            stream, 1, (float*)out, (float8_e4m3_t*)a, (float8_e5m2_t*)b, (S*)sa, (S*)sb, (float*)nullptr);
    case 4: return run<&RunTMATMUL_MX<float4_e2m1x2_t, float4_e2m1x2_t, 40, 128, 60, Layout::MX_A_ND, Layout::MX_B_DN, false>>(
            stream, 1, (float*)out, (float4_e2m1x2_t*)a, (float4_e2m1x2_t*)b, (S*)sa, (S*)sb, (float*)nullptr);
    case 5: return run<&RunTMATMUL_MX<float4_e2m1x2_t, float4_e2m1x2_t, 32, 256, 64, Layout::MX_A_ZZ, Layout::MX_B_NN, true>>(
            stream, 1, (float*)out, (float4_e2m1x2_t*)a, (float4_e2m1x2_t*)b, (S*)sa, (S*)sb, (float*)bias);
    default: return -1;
    }
}

// matmul, then TSTORE through the fix-pipe quantiser: a scalar word, or one word per column from a Scaling tile
template <typename OutT, typename AccT, typename InT, int validM, int validK, int validN, bool VECTOR, bool RELU>
__global__ AICORE void RunTMATMUL_QUANT(__gm__ OutT* out, __gm__ InT* src0, __gm__ InT* src1, __gm__ uint64_t* words)
{
    constexpr int blockAlign = (sizeof(InT) == 1) ? 32 : 16;
    constexpr int M = CeilAlign<int>(validM, 16), N = CeilAlign<int>(validN, blockAlign), K = CeilAlign<int>(validK, blockAlign);
    GlobalTensor<InT, TileShape2D<InT, validM, validK>, BaseShape2D<InT, validM, validK>> aGlobal(src0);
    GlobalTensor<InT, TileShape2D<InT, validK, validN>, BaseShape2D<InT, validK, validN>> bGlobal(src1);
    GlobalTensor<OutT, TileShape2D<OutT, validM, validN>, BaseShape2D<OutT, validM, validN>> outGlobal(out);
    GlobalTensor<uint64_t, TileShape2D<uint64_t, 1, validN>, BaseShape2D<uint64_t, 1, validN>> wordsGlobal(words);
    Tile<TileType::Mat, InT, M, K, BLayout::ColMajor, validM, validK, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, InT, K, N, BLayout::ColMajor, validK, validN, SLayout::RowMajor, 512> bMat;
    TileLeft<InT, M, K, validM, validK> aTile;
    TileRight<InT, K, N, validK, validN> bTile;
    TileAcc<AccT, M, N, validM, validN> cTile;
    Tile<TileType::Scaling, uint64_t, 1, N, BLayout::RowMajor, 1, validN> fpTile;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    TASSIGN(fpTile, 0x0);
    TLOAD(aMat, aGlobal);
    TLOAD(bMat, bGlobal);
    TMOV(aTile, aMat);
    TMOV(bTile, bMat);
    TMATMUL(cTile, aTile, bTile);
    constexpr ReluPreMode relu = RELU ? ReluPreMode::NormalRelu : ReluPreMode::NoRelu;
    if constexpr (VECTOR) {
        TLOAD(fpTile, wordsGlobal);
        TSTORE<decltype(cTile), decltype(outGlobal), decltype(fpTile), AtomicType::AtomicNone, relu>(outGlobal, cTile, fpTile);
    } else {
        TSTORE<decltype(cTile), decltype(outGlobal), AtomicType::AtomicNone, relu>(outGlobal, cTile, words[0]);
    }
}

// ---- TQUANT / TDEQUANT on Vec tiles ----------------------------------------------------------------------------------
template <typename SrcT, typename DstT, int R, int C, QuantType QT, QuantScaleAlg ALG>
__global__ AICORE void RunTQUANT_MX(__gm__ DstT* dst, __gm__ uint8_t* exp, __gm__ float* max, __gm__ float* scaling, __gm__ SrcT* src)
{
    constexpr int G = R * C / 32;
    using SrcTile = Tile<TileType::Vec, SrcT, R, C, BLayout::RowMajor, R, C>;
    using DstTile = Tile<TileType::Vec, DstT, R, C, BLayout::RowMajor, R, C>;
    using ExpTile = Tile<TileType::Vec, uint8_t, 1, G, BLayout::RowMajor, 1, G>;
    using FlatTile = Tile<TileType::Vec, float, 1, G, BLayout::RowMajor, 1, G>;
    SrcTile srcTile;
    DstTile dstTile;
    ExpTile expTile;
    FlatTile maxTile, scalingTile;
    constexpr int a1 = CeilAlign<int>(SrcTile::Bytes, 32), a2 = a1 + CeilAlign<int>(DstTile::Bytes, 32),
                  a3 = a2 + CeilAlign<int>(ExpTile::Bytes, 32), a4 = a3 + CeilAlign<int>(FlatTile::Bytes, 32);
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, a1);
    TASSIGN(expTile, a2);
    TASSIGN(maxTile, a3);
    TASSIGN(scalingTile, a4);
    GlobalTensor<SrcT, TileShape2D<SrcT, R, C>, BaseShape2D<SrcT, R, C>> srcGlobal(src);
    GlobalTensor<DstT, TileShape2D<DstT, R, C>, BaseShape2D<DstT, R, C>> dstGlobal(dst);
    GlobalTensor<uint8_t, TileShape2D<uint8_t, 1, G>, BaseShape2D<uint8_t, 1, G>> expGlobal(exp);
    GlobalTensor<float, TileShape2D<float, 1, G>, BaseShape2D<float, 1, G>> maxGlobal(max), scalingGlobal(scaling);
    TLOAD(srcTile, srcGlobal);
    TQUANT<QT, DstTile, SrcTile, ExpTile, FlatTile, FlatTile, ALG>(dstTile, srcTile, &expTile, &maxTile, &scalingTile);
    TSTORE(dstGlobal, dstTile);
    TSTORE(expGlobal, expTile);
    TSTORE(maxGlobal, maxTile);
    TSTORE(scalingGlobal, scalingTile);
}

// NZ store mode: the exponents are written twice, row-major in exp and in 16 x 2 boxes in exp_zz (stored to `max`'s
// buffer reinterpreted as bytes: the launcher has no separate pointer for it)
template <typename SrcT, int R, int C>
__global__ AICORE void RunTQUANT_MX_NZ(__gm__ float8_e4m3_t* dst, __gm__ uint8_t* exp, __gm__ uint8_t* exp_zz, __gm__ float* scaling, __gm__ SrcT* src)
{
    constexpr int G = R * C / 32;
    using SrcTile = Tile<TileType::Vec, SrcT, R, C, BLayout::RowMajor, R, C>;
    using DstTile = Tile<TileType::Vec, float8_e4m3_t, R, C, BLayout::RowMajor, R, C>;
    using ExpTile = Tile<TileType::Vec, uint8_t, 1, G, BLayout::RowMajor, 1, G>;
    using FlatTile = Tile<TileType::Vec, float, 1, G, BLayout::RowMajor, 1, G>;
    SrcTile srcTile;
    DstTile dstTile;
    ExpTile expTile, zzTile;
    FlatTile maxTile, scalingTile;
    constexpr int a1 = CeilAlign<int>(SrcTile::Bytes, 32), a2 = a1 + CeilAlign<int>(DstTile::Bytes, 32),
                  a3 = a2 + CeilAlign<int>(ExpTile::Bytes, 32), a4 = a3 + CeilAlign<int>(ExpTile::Bytes, 32),
                  a5 = a4 + CeilAlign<int>(FlatTile::Bytes, 32);
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, a1);
    TASSIGN(expTile, a2);
    TASSIGN(zzTile, a3);
    TASSIGN(maxTile, a4);
    TASSIGN(scalingTile, a5);
    GlobalTensor<SrcT, TileShape2D<SrcT, R, C>, BaseShape2D<SrcT, R, C>> srcGlobal(src);
    GlobalTensor<float8_e4m3_t, TileShape2D<float8_e4m3_t, R, C>, BaseShape2D<float8_e4m3_t, R, C>> dstGlobal(dst);
    GlobalTensor<uint8_t, TileShape2D<uint8_t, 1, G>, BaseShape2D<uint8_t, 1, G>> expGlobal(exp), zzGlobal(exp_zz);
    GlobalTensor<float, TileShape2D<float, 1, G>, BaseShape2D<float, 1, G>> scalingGlobal(scaling);
    TLOAD(srcTile, srcGlobal);
    TQUANT<QuantType::MXFP8, VecStoreMode::NZ>(dstTile, srcTile, &expTile, &maxTile, &scalingTile, &zzTile);
    TSTORE(dstGlobal, dstTile);
    TSTORE(expGlobal, expTile);
    TSTORE(zzGlobal, zzTile);
    TSTORE(scalingGlobal, scalingTile);
}

// column-grouped form: 32 consecutive rows of one column share an exponent; exp / max / scaling are [R / 32][C]
template <typename DstT, int R, int C, MxQuantAlg ALG>
__global__ AICORE void RunTQUANT_MX_DN(__gm__ DstT* dst, __gm__ uint8_t* exp, __gm__ float* max, __gm__ float* scaling, __gm__ float* src)
{
    constexpr int G = R / 32 * C;
    using SrcTile = Tile<TileType::Vec, float, R, C, BLayout::RowMajor, R, C>;
    using DstTile = Tile<TileType::Vec, DstT, R, C, BLayout::RowMajor, R, C>;
    using ExpTile = Tile<TileType::Vec, uint8_t, R / 32, C, BLayout::RowMajor, R / 32, C>;
    using FlatTile = Tile<TileType::Vec, float, R / 32, C, BLayout::RowMajor, R / 32, C>;
    SrcTile srcTile;
    DstTile dstTile;
    ExpTile expTile;
    FlatTile maxTile, scalingTile;
    constexpr int a1 = CeilAlign<int>(SrcTile::Bytes, 32), a2 = a1 + CeilAlign<int>(DstTile::Bytes, 32),
                  a3 = a2 + CeilAlign<int>(ExpTile::Bytes, 32), a4 = a3 + CeilAlign<int>(FlatTile::Bytes, 32);
    static_assert(G > 0, "at least one group");
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, a1);
    TASSIGN(expTile, a2);
    TASSIGN(maxTile, a3);
    TASSIGN(scalingTile, a4);
    GlobalTensor<float, TileShape2D<float, R, C>, BaseShape2D<float, R, C>> srcGlobal(src);
    GlobalTensor<DstT, TileShape2D<DstT, R, C>, BaseShape2D<DstT, R, C>> dstGlobal(dst);
    GlobalTensor<uint8_t, TileShape2D<uint8_t, R / 32, C>, BaseShape2D<uint8_t, R / 32, C>> expGlobal(exp);
    GlobalTensor<float, TileShape2D<float, R / 32, C>, BaseShape2D<float, R / 32, C>> maxGlobal(max), scalingGlobal(scaling);
    TLOAD(srcTile, srcGlobal);
    TQUANT<0, ALG>(dstTile, srcTile, &expTile, &maxTile, &scalingTile);
    TSTORE(dstGlobal, dstTile);
    TSTORE(expGlobal, expTile);
    TSTORE(maxGlobal, maxTile);
    TSTORE(scalingGlobal, scalingTile);
}

template <int R, int C, bool ASYM>
__global__ AICORE void RunTQUANT_INT8(__gm__ uint8_t* dst, __gm__ float* src, __gm__ float* scale, __gm__ float* offset)
{
    using SrcTile = Tile<TileType::Vec, float, R, C, BLayout::RowMajor, R, C>;
    using DstTile = Tile<TileType::Vec, uint8_t, R, C, BLayout::RowMajor, R, C>;
    using ParaTile = Tile<TileType::Vec, float, R, 8, BLayout::RowMajor, R, 1>;  // one value per row
    SrcTile srcTile;
    DstTile dstTile;
    ParaTile scaleTile, offsetTile;
    TASSIGN(srcTile, 0x0);
    TASSIGN(dstTile, SrcTile::Bytes);
    TASSIGN(scaleTile, SrcTile::Bytes + DstTile::Bytes);
    TASSIGN(offsetTile, SrcTile::Bytes + DstTile::Bytes + ParaTile::Bytes);
    GlobalTensor<float, TileShape2D<float, R, C>, BaseShape2D<float, R, C>> srcGlobal(src);
    GlobalTensor<uint8_t, TileShape2D<uint8_t, R, C>, BaseShape2D<uint8_t, R, C>> dstGlobal(dst);
    GlobalTensor<float, TileShape2D<float, R, 1>, BaseShape2D<float, R, 1>> scaleGlobal(scale), offsetGlobal(offset);
    TLOAD(srcTile, srcGlobal);
    TLOAD(scaleTile, scaleGlobal);
    if constexpr (ASYM) {
        TLOAD(offsetTile, offsetGlobal);
        TQUANT<QuantType::INT8_ASYM>(dstTile, srcTile, scaleTile, &offsetTile);
    } else {
        TQUANT<QuantType::INT8_SYM>(dstTile, srcTile, scaleTile);
    }
    TSTORE(dstGlobal, dstTile);
}

template <typename SrcT, int R, int C>
__global__ AICORE void RunTDEQUANT(__gm__ float* dst, __gm__ SrcT* src, __gm__ float* scale, __gm__ float* offset)
{
    using SrcTile = Tile<TileType::Vec, SrcT, R, C, BLayout::RowMajor, R, C>;
    using DstTile = Tile<TileType::Vec, float, R, C, BLayout::RowMajor, R, C>;
    using ParaTile = Tile<TileType::Vec, float, R, 8, BLayout::RowMajor, R, 1>;
    SrcTile srcTile;
    DstTile dstTile;
    ParaTile scaleTile, offsetTile;
    TASSIGN(dstTile, 0x0);
    TASSIGN(srcTile, DstTile::Bytes);
    TASSIGN(scaleTile, DstTile::Bytes + CeilAlign<int>(SrcTile::Bytes, 32));
    TASSIGN(offsetTile, DstTile::Bytes + CeilAlign<int>(SrcTile::Bytes, 32) + ParaTile::Bytes);
    GlobalTensor<SrcT, TileShape2D<SrcT, R, C>, BaseShape2D<SrcT, R, C>> srcGlobal(src);
    GlobalTensor<float, TileShape2D<float, R, C>, BaseShape2D<float, R, C>> dstGlobal(dst);
    GlobalTensor<float, TileShape2D<float, R, 1>, BaseShape2D<float, R, 1>> scaleGlobal(scale), offsetGlobal(offset);
    TLOAD(srcTile, srcGlobal);
    TLOAD(scaleTile, scaleGlobal);
    TLOAD(offsetTile, offsetGlobal);
    TDEQUANT(dstTile, srcTile, scaleTile, offsetTile);
    TSTORE(dstGlobal, dstTile);
}

// quant cases: 1-4: f32 16x64 -> OCP-FP8, NV-FP8, OCP-FP4, NV-FP4     5: bf16 8x128 -> OCP-FP4     6: half 8x128 -> OCP-FP8
//              7, 8: f32 64x16 grouped along columns -> OCP-FP8, NV-FP4     9: half 16x128 -> OCP-FP8, NZ store mode
//              10: INT8 sym 16x64   11: INT8 asym 16x64    20: TDEQUANT int8 16x64    21: TDEQUANT int32 8x32
extern "C" int pto_kernels_launch_quant(int id, void* dst, void* exp, void* max, void* scaling, void* src, void* scale, void* offset, void* stream)
{
    using F8 = float8_e4m3_t;
    using F4 = float4_e2m1x2_t;
    switch (id) {
    case 1: return run<&RunTQUANT_MX<float, F8, 16, 64, QuantType::MXFP8, QuantScaleAlg::OCP>>(stream, 1, (F8*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 2: return run<&RunTQUANT_MX<float, F8, 16, 64, QuantType::MXFP8, QuantScaleAlg::NV>>(stream, 1, (F8*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 3: return run<&RunTQUANT_MX<float, F4, 16, 64, QuantType::MXFP4_E2M1, QuantScaleAlg::OCP>>(stream, 1, (F4*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 4: return run<&RunTQUANT_MX<float, F4, 16, 64, QuantType::MXFP4_E2M1, QuantScaleAlg::NV>>(stream, 1, (F4*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 5: return run<&RunTQUANT_MX<bfloat16_t, F4, 8, 128, QuantType::MXFP4_E2M1, QuantScaleAlg::OCP>>(stream, 1, (F4*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (bfloat16_t*)src);
    case 6: return run<&RunTQUANT_MX<half, F8, 8, 128, QuantType::MXFP8, QuantScaleAlg::OCP>>(stream, 1, (F8*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (half*)src);
    case 7: return run<&RunTQUANT_MX_DN<F8, 64, 16, MxQuantAlg::OcpMxFp8E4M3>>(stream, 1, (F8*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 8: return run<&RunTQUANT_MX_DN<F4, 64, 16, MxQuantAlg::NvMxFp4E2M1>>(stream, 1, (F4*)dst, (uint8_t*)exp, (float*)max, (float*)scaling, (float*)src);
    case 9: return run<&RunTQUANT_MX_NZ<half, 16, 128>>(stream, 1, (F8*)dst, (uint8_t*)exp, (uint8_t*)max, (float*)scaling, (half*)src);
    case 10: return run<&RunTQUANT_INT8<16, 64, false>>(stream, 1, (uint8_t*)dst, (float*)src, (float*)scale, (float*)offset);
    case 11: return run<&RunTQUANT_INT8<16, 64, true>>(stream, 1, (uint8_t*)dst, (float*)src, (float*)scale, (float*)offset);
    case 20: return run<&RunTDEQUANT<int8_t, 16, 64>>(stream, 1, (float*)dst, (int8_t*)src, (float*)scale, (float*)offset);
    case 21: return run<&RunTDEQUANT<int32_t, 8, 32>>(stream, 1, (float*)dst, (int32_t*)src, (float*)scale, (float*)offset);
    default: return -1;
    }
}

// store-quant cases: 1: f16 -> f32 acc -> int8, scalar word     2: f16 -> f32 acc -> uint8, per-column words, relu
//                    3: int8 -> i32 acc -> f16 (dequant), per-column words     4: int8 -> i32 acc -> int8 (requant), scalar
//                    5: f16 -> f32 acc -> bf16, scalar word     6: int8 -> i32 acc -> bf16, per-column words, relu
//                    7: int8 -> i32 acc -> int16 (shift mode), scalar word     8: the same, per-column words, relu
extern "C" int pto_kernels_launch_store_quant(int id, void* out, void* a, void* b, void* words, void* stream)
{
    switch (id) {
    case 1: return run<&RunTMATMUL_QUANT<int8_t, float, half, 40, 50, 60, false, false>>(stream, 1, (int8_t*)out, (half*)a, (half*)b, (uint64_t*)words);
    case 2: return run<&RunTMATMUL_QUANT<uint8_t, float, half, 33, 64, 70, true, true>>(stream, 1, (uint8_t*)out, (half*)a, (half*)b, (uint64_t*)words);
    case 3: return run<&RunTMATMUL_QUANT<half, int32_t, int8_t, 24, 96, 40, true, false>>(stream, 1, (half*)out, (int8_t*)a, (int8_t*)b, (uint64_t*)words);
    case 4: return run<&RunTMATMUL_QUANT<int8_t, int32_t, int8_t, 24, 96, 40, false, false>>(stream, 1, (int8_t*)out, (int8_t*)a, (int8_t*)b, (uint64_t*)words);
    case 5: return run<&RunTMATMUL_QUANT<bfloat16_t, float, half, 40, 50, 60, false, false>>(stream, 1, (bfloat16_t*)out, (half*)a, (half*)b, (uint64_t*)words);
    case 6: return run<&RunTMATMUL_QUANT<bfloat16_t, int32_t, int8_t, 24, 96, 40, true, true>>(stream, 1, (bfloat16_t*)out, (int8_t*)a, (int8_t*)b, (uint64_t*)words);
    case 7: return run<&RunTMATMUL_QUANT<int16_t, int32_t, int8_t, 24, 96, 40, false, false>>(stream, 1, (int16_t*)out, (int8_t*)a, (int8_t*)b, (uint64_t*)words);
    case 8: return run<&RunTMATMUL_QUANT<int16_t, int32_t, int8_t, 24, 96, 40, true, true>>(stream, 1, (int16_t*)out, (int8_t*)a, (int8_t*)b, (uint64_t*)words);
    default: return -1;
    }
}

extern "C" int pto_kernels_status() { return pto::amd::device_status(); }
