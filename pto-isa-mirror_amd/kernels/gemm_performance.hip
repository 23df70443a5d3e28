// A tuned GEMM written in the PTO tile ISA for the gfx950 backend: C[M, N] = A[M, K] . B[K, N], A row-major (ND), B
// column-major (the DN view of [N][K] memory), fp32 accumulation, C row-major.  The program has the shape of the
// reference's performance kernel (kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp:69-131, 170-235):
// every core owns one baseM x baseN tile of C, walks K in panels of baseK * stepK that TLOAD double-buffers in L1,
// slices each panel into baseK pieces with TEXTRACT, accumulates with TMATMUL / TMATMUL_ACC and drains with one TSTORE.
//
// What is sized for this backend rather than for an Ascend core:
//   * a core is a workgroup of 512 threads (8 waves), and the L1 region takes most of the CU's 160 KiB of LDS: two panels
//     of A and two of B;
//   * Left / Right tiles extracted from those panels are windows onto them, so L0A / L0B need no bytes of their own;
//   * 20 KiB of fix-pipe staging let TSTORE turn the accumulator blocks into whole 64-byte rows of bf16;
//   * a core executes its tile instructions in program order, so the copy-in of panel p + 1 is issued *before* the
//     TMATMULs of panel p (TLOAD only starts the copies; the TEXTRACT of the next iteration waits for them), where the
//     reference issues it in the same iteration and lets the MTE2 queue run ahead.  Of the event flags of the reference
//     program one is left: wait_flag(PIPE_MTE2, PIPE_MTE1) names the two tiles of a panel, so that their arrival costs
//     one barrier instead of one per tile; the others have nothing left to order and are not written out.
#define PTO_AMD_THREADS 512
#define PTO_AMD_L1_BYTES (128 * 1024)
#define PTO_AMD_L0A_BYTES (1 * 1024)
#define PTO_AMD_L0B_BYTES (1 * 1024)
#define PTO_AMD_UB_BYTES (1 * 1024)
#define PTO_AMD_BIAS_BYTES (1 * 1024)
#define PTO_AMD_FB_BYTES (1 * 1024)
#define PTO_AMD_L0S_BYTES (1 * 1024)
// every TLOAD below follows the TEXTRACT of a freshly loaded panel and targets the buffer whose last readers came before it
#define PTO_AMD_TLOAD_AFTER_ACQUIRE
#define PTO_AMD_STAGE_BYTES (8 * 32 * (64 + 16))  // a band of 32 rows x (64 + 16) bytes per wave: 16-bit results leave as whole rows
#include <pto/pto-inst.hpp>

using namespace pto;

// Which tile of C a core owns.  Consecutive core ids land on different XCDs (8 of them, each with its own L2), so ids
// are first regrouped per XCD and then walked groupM tile rows at a time: an XCD's cores then share a compact block of
// tiles and with it their A and B panels.
template <int tilesM, int tilesN, int groupM>
AICORE inline void OwnTile(int& tm, int& tn)
{
    constexpr int cores = tilesM * tilesN;
    int id = (int)get_block_idx();
    if constexpr (cores % 8 == 0)
        id = (id & 7) * (cores / 8) + (id >> 3);
    constexpr int perGroup = groupM * tilesN;
    const int firstM = (id / perGroup) * groupM;
    const int rows = (tilesM - firstM) < groupM ? (tilesM - firstM) : groupM;
    tm = firstM + (id % perGroup) % rows;
    tn = (id % perGroup) / rows;
}

template <typename OutT, typename InT, int M, int K, int N, int baseM, int baseN, int baseK, int stepK>
__global__ AICORE void GemmPerformance(__gm__ OutT* out, __gm__ InT* a, __gm__ InT* b)
{
    constexpr int panelK = baseK * stepK, panels = K / panelK;
    static_assert(M % baseM == 0 && N % baseN == 0 && K % panelK == 0, "whole tiles and panels only");

    // A panel [baseM, panelK] of the row-major A; B panel [panelK, baseN] of the column-major B
    using PanelShapeA = TileShape2D<InT, baseM, panelK, Layout::ND>;
    using WholeStrideA = BaseShape2D<InT, M, K, Layout::ND>;
    using GlobalA = GlobalTensor<InT, PanelShapeA, WholeStrideA, Layout::ND>;
    using PanelShapeB = TileShape2D<InT, panelK, baseN, Layout::DN>;
    using WholeStrideB = BaseShape2D<InT, K, N, Layout::DN>;
    using GlobalB = GlobalTensor<InT, PanelShapeB, WholeStrideB, Layout::DN>;
    using TileShapeC = TileShape2D<OutT, baseM, baseN, Layout::ND>;
    using WholeStrideC = BaseShape2D<OutT, M, N, Layout::ND>;
    using GlobalC = GlobalTensor<OutT, TileShapeC, WholeStrideC, Layout::ND>;

    using TileMatA = Tile<TileType::Mat, InT, baseM, panelK, BLayout::ColMajor, baseM, panelK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, InT, panelK, baseN, BLayout::RowMajor, panelK, baseN, SLayout::ColMajor>;
    using LeftTile = TileLeft<InT, baseM, baseK, baseM, baseK>;
    using RightTile = TileRight<InT, baseK, baseN, baseK, baseN>;
    using ResTile = TileAcc<float, baseM, baseN, baseM, baseN>;

    TileMatA aMat[2];
    TileMatB bMat[2];
    LeftTile aTile;
    RightTile bTile;
    ResTile cTile;
    constexpr uint32_t bytesA = baseM * panelK * sizeof(InT), bytesB = panelK * baseN * sizeof(InT);
    TASSIGN(aMat[0], 0x0);
    TASSIGN(aMat[1], bytesA);
    TASSIGN(bMat[0], 2 * bytesA);
    TASSIGN(bMat[1], 2 * bytesA + bytesB);
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);

    int tm, tn;
    OwnTile<M / baseM, N / baseN, 4>(tm, tn);
    __gm__ InT* aPanel = a + (size_t)tm * baseM * K;  // rows of A this core reads
    __gm__ InT* bPanel = b + (size_t)tn * baseN * K;  // columns of B (rows of the [N][K] memory)

    // one panel: make its slices the operands, start the copy-in of the next panel into the other L1 slot, multiply
    auto panel = [&](auto slot, int p) __attribute__((always_inline)) {
        constexpr int cur = decltype(slot)::value, nxt = cur ^ 1;
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0, aMat[cur], bMat[cur]);  // the panel has landed: one wait for both tiles
        for (int s = 0; s < stepK; ++s) {
            TEXTRACT(aTile, aMat[cur], 0, s * baseK);
            TEXTRACT(bTile, bMat[cur], s * baseK, 0);
            if (s == 0 && p + 1 < panels) {
                GlobalA gmA(aPanel + (size_t)(p + 1) * panelK);
                GlobalB gmB(bPanel + (size_t)(p + 1) * panelK);
                TLOAD(aMat[nxt], gmA);
                TLOAD(bMat[nxt], gmB);
            }
            if (p == 0 && s == 0)
                TMATMUL(cTile, aTile, bTile);
            else
                TMATMUL_ACC(cTile, cTile, aTile, bTile);
        }
    };

    {
        GlobalA gmA(aPanel);
        GlobalB gmB(bPanel);
        TLOAD(aMat[0], gmA);
        TLOAD(bMat[0], gmB);
    }
    for (int p = 0; p < panels; p += 2) {
        panel(std::integral_constant<int, 0>{}, p);
        if (p + 1 < panels)
            panel(std::integral_constant<int, 1>{}, p + 1);
    }

    GlobalC gmC(out + (size_t)tm * baseM * N + (size_t)tn * baseN);
    TSTORE(gmC, cTile);
}

// ---- launchers ------------------------------------------------------------------------------------------------------
// id 0: bf16 4096^3 -> bf16 (256 x 256 tiles, K panels of 64: one core per CU of a 256-CU part)
// id 1: bf16 4096^3 -> f32
// id 2: f16 1024 x 1024 x 512 -> f32 (16 cores; a small case for parity tests)
template <typename OutT, typename InT, int M, int K, int N, int baseM, int baseN, int baseK, int stepK>
static int run(void* out, void* a, void* b, void* stream)
{
    constexpr int cores = (M / baseM) * (N / baseN);
    return pto::amd::launch<&GemmPerformance<OutT, InT, M, K, N, baseM, baseN, baseK, stepK>>(cores, stream, (OutT*)out, (InT*)a, (InT*)b);
}

extern "C" int pto_gemm_performance(int id, void* out, void* a, void* b, void* stream)
{
    switch (id) {
    case 0: return run<bfloat16_t, bfloat16_t, 4096, 4096, 4096, 256, 256, 64, 1>(out, a, b, stream);
    case 1: return run<float, bfloat16_t, 4096, 4096, 4096, 256, 256, 64, 1>(out, a, b, stream);
    case 2: return run<float, half, 1024, 512, 1024, 256, 256, 64, 1>(out, a, b, stream);
    default: return -1;
    }
}

extern "C" int pto_gemm_performance_status() { return pto::amd::device_status(); }
