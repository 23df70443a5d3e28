// The tiled GEMM of the reference's CPU-simulator demo (demos/cpu/gemm_demo/gemm_demo.cpp:83-121) at the size of
// configs[0]: C[512, 512] = A[512, 512] . B[512, 512], fp16 inputs, fp32 result, A and B row-major, one core per
// 128 x 128 tile of C, K walked in slabs of 64 through TLOAD -> TMOV -> TMATMUL / TMATMUL_ACC, one TSTORE per core.
// B arrives row-major ([K][N]), so its slab sits in L1 with N contiguous and the TMOV into the Right tile transposes
// (a copy into L0B); A's slab becomes a window.  The copy-in of slab s + 1 is issued before the TMATMUL of slab s.
#define PTO_AMD_THREADS 256
#define PTO_AMD_L1_BYTES (64 * 1024)
#define PTO_AMD_L0A_BYTES (16 * 1024)
#define PTO_AMD_L0B_BYTES (16 * 1024)
#define PTO_AMD_UB_BYTES (1 * 1024)
#define PTO_AMD_BIAS_BYTES (1 * 1024)
#define PTO_AMD_FB_BYTES (1 * 1024)
#define PTO_AMD_L0S_BYTES (1 * 1024)
#define PTO_AMD_STAGE_BYTES (4 * 32 * (128 + 16))  // 4 waves x a band of 32 rows x (128 + 16) bytes: fp32 results leave as whole rows
#include <pto/pto-inst.hpp>

using namespace pto;

template <typename OutT, typename InT, int M, int K, int N, int BM, int BN, int BK>
__global__ AICORE void RunTiledGemm(__gm__ OutT* out, __gm__ InT* a, __gm__ InT* b)
{
    constexpr int tilesN = N / BN, slabs = K / BK;
    const int tile = (int)get_block_idx();
    const int tm = tile / tilesN, tn = tile % tilesN;

    using GlobalA = GlobalTensor<InT, TileShape2D<InT, BM, BK, Layout::ND>, BaseShape2D<InT, M, K, Layout::ND>, Layout::ND>;
    using GlobalB = GlobalTensor<InT, TileShape2D<InT, BK, BN, Layout::ND>, BaseShape2D<InT, K, N, Layout::ND>, Layout::ND>;
    using GlobalC = GlobalTensor<OutT, TileShape2D<OutT, BM, BN, Layout::ND>, BaseShape2D<OutT, M, N, Layout::ND>, Layout::ND>;
    using MatA = Tile<TileType::Mat, InT, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, InT, BK, BN, BLayout::ColMajor, BK, BN, SLayout::RowMajor, 512>;

    MatA aMat[2];
    MatB bMat[2];
    TileLeft<InT, BM, BK> aTile;
    TileRight<InT, BK, BN> bTile;
    TileAcc<float, BM, BN> cTile;
    constexpr uint32_t bytesA = BM * BK * sizeof(InT), bytesB = BK * BN * sizeof(InT);
    TASSIGN(aMat[0], 0x0);
    TASSIGN(aMat[1], bytesA);
    TASSIGN(bMat[0], 2 * bytesA);
    TASSIGN(bMat[1], 2 * bytesA + bytesB);
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);

    __gm__ InT* aRows = a + (size_t)tm * BM * K;
    __gm__ InT* bCols = b + (size_t)tn * BN;
    auto slab = [&](auto slot, int s) __attribute__((always_inline)) {
        constexpr int cur = decltype(slot)::value, nxt = cur ^ 1;
        TMOV(aTile, aMat[cur]);
        TMOV(bTile, bMat[cur]);
        if (s + 1 < slabs) {
            GlobalA aGlobal(aRows + (size_t)(s + 1) * BK);
            GlobalB bGlobal(bCols + (size_t)(s + 1) * BK * N);
            TLOAD(aMat[nxt], aGlobal);
            TLOAD(bMat[nxt], bGlobal);
        }
        if (s == 0)
            TMATMUL(cTile, aTile, bTile);
        else
            TMATMUL_ACC(cTile, cTile, aTile, bTile);
    };
    {
        GlobalA aGlobal(aRows);
        GlobalB bGlobal(bCols);
        TLOAD(aMat[0], aGlobal);
        TLOAD(bMat[0], bGlobal);
    }
    for (int s = 0; s < slabs; s += 2) {
        slab(std::integral_constant<int, 0>{}, s);
        if (s + 1 < slabs)
            slab(std::integral_constant<int, 1>{}, s + 1);
    }
    GlobalC cGlobal(out + (size_t)tm * BM * N + (size_t)tn * BN);
    TSTORE(cGlobal, cTile);
}

// id 0: configs[0], fp16 512^3 -> fp32 with 128 x 128 x 64 tiles (16 cores)     id 1: the same product with 64 x 64 tiles (64 cores)
extern "C" int pto_gemm_tiled(int id, void* out, void* a, void* b, void* stream)
{
    switch (id) {
    case 0: return pto::amd::launch<&RunTiledGemm<float, half, 512, 512, 512, 128, 128, 64>>(16, stream, (float*)out, (half*)a, (half*)b);
    case 1: return pto::amd::launch<&RunTiledGemm<float, half, 512, 512, 512, 64, 64, 64>>(64, stream, (float*)out, (half*)a, (half*)b);
    default: return -1;
    }
}

extern "C" int pto_gemm_tiled_status() { return pto::amd::device_status(); }
