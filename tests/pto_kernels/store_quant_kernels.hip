// The reference's tstore_quant case list (tests/cpu/st/testcase/tstore_quant/main.cpp:112-130) as PTO-style kernels: a
// Vec tile of float / int32 values is loaded from a 5-D global tensor (ND: rows = g0 g1 g2 g3, cols = g4; DN: rows = g3,
// cols = g0 g1 g2 g4, stored column by column) and leaves through the quantising TSTORE -- one scalar word, or one word
// per column from a one-row Vec tile of 64-bit elements (TSTORE_FP).  A large UB: the tiles are up to 276 x 48 int32.
#define PTO_AMD_L1_BYTES (16 * 1024)
#define PTO_AMD_L0A_BYTES (8 * 1024)
#define PTO_AMD_L0B_BYTES (8 * 1024)
#define PTO_AMD_UB_BYTES (96 * 1024)
#include <pto/pto-inst.hpp>
#include <pto/common/pto_tile.hpp>
#include <pto/common/constants.hpp>

using namespace pto;

constexpr int RoundUp(int a, int b) { return (a + b - 1) / b * b; }

template <typename DstT, typename SrcT, bool DN, int g0, int g1, int g2, int g3, int g4, bool perColumn, bool relu>
__global__ AICORE void RunStoreQuant(__gm__ DstT* out, __gm__ SrcT* src, __gm__ uint64_t* words)
{
    constexpr int block = 32 / (int)sizeof(SrcT);
    constexpr int validRow = DN ? g3 : g0 * g1 * g2 * g3;
    constexpr int validCol = DN ? g0 * g1 * g2 * g4 : g4;
    constexpr int Rows = DN ? RoundUp(validRow, block) : validRow;
    constexpr int Cols = DN ? validCol : RoundUp(validCol, block);
    using Shape5 = Shape<g0, g1, g2, g3, g4>;
    using Stride5 = std::conditional_t<DN, Stride<g1 * g2 * g3 * g4, g2 * g3 * g4, g3 * g4, 1, g3>,
                                       Stride<g1 * g2 * g3 * g4, g2 * g3 * g4, g3 * g4, g4, 1>>;
    constexpr Layout L = DN ? Layout::DN : Layout::ND;
    using GlobalDst = GlobalTensor<DstT, Shape5, Stride5, L>;
    using GlobalSrc = GlobalTensor<SrcT, Shape5, Stride5, L>;
    using TileData = Tile<TileType::Vec, SrcT, Rows, Cols, DN ? BLayout::ColMajor : BLayout::RowMajor, -1, -1>;
    constexpr ReluPreMode mode = relu ? ReluPreMode::NormalRelu : ReluPreMode::NoRelu;

    TileData tile(validRow, validCol);
    TASSIGN(tile, 0x0);
    GlobalDst dstGlobal(out);
    GlobalSrc srcGlobal(src);
    TLOAD(tile, srcGlobal);
    set_flag(PIPE_MTE2, PIPE_MTE3, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE3, EVENT_ID0);
    if constexpr (perColumn) {
        GlobalTensor<uint64_t, Shape<1, 1, 1, 1, validCol>, Stride<validCol, validCol, validCol, validCol, 1>> wordsGlobal(words);
        using WordTile = Tile<TileType::Vec, uint64_t, 1, Cols, BLayout::RowMajor, 1, validCol>;
        WordTile wordTile;
        TASSIGN(wordTile, 0x400 + Rows * Cols * sizeof(SrcT));
        TLOAD(wordTile, wordsGlobal);
        TSTORE_FP<TileData, GlobalDst, WordTile, AtomicType::AtomicNone, mode>(dstGlobal, tile, wordTile);
    } else {
        TSTORE<TileData, GlobalDst, AtomicType::AtomicNone, mode>(dstGlobal, tile, words[0]);
    }
}

template <auto K, typename... A>
static int run(void* stream, A... a)
{
    return pto::amd::launch<K>(1, stream, a...);
}

// Case ids are the reference's (ND_1 ... ND_10); `saturate` is what its cases name saturate_inf: bit 48 of the task cookie.
extern "C" int pto_store_quant_launch(int id, void* out, void* src, void* words, int saturate, void* stream)
{
    if (const int rc = pto::amd::set_task_cookie(saturate ? (1ull << 48) : 0); rc != 0)
        return rc;
    auto* w = (uint64_t*)words;
    switch (id) {
    case 1: return run<&RunStoreQuant<int8_t, float, false, 1, 1, 1, 2, 128, true, true>>(stream, (int8_t*)out, (float*)src, w);
    case 2: return run<&RunStoreQuant<int16_t, int32_t, false, 1, 2, 1, 23, 121, true, false>>(stream, (int16_t*)out, (int32_t*)src, w);
    case 3: return run<&RunStoreQuant<int8_t, int32_t, false, 2, 2, 3, 23, 47, true, true>>(stream, (int8_t*)out, (int32_t*)src, w);
    case 4: return run<&RunStoreQuant<half, float, true, 1, 1, 1, 4, 21, false, true>>(stream, (half*)out, (float*)src, w);
    case 5: return run<&RunStoreQuant<half, float, true, 3, 1, 1, 1, 124, false, false>>(stream, (half*)out, (float*)src, w);
    case 6: return run<&RunStoreQuant<int8_t, int32_t, true, 2, 1, 2, 32, 32, false, false>>(stream, (int8_t*)out, (int32_t*)src, w);
    case 7: return run<&RunStoreQuant<half, float, true, 1, 1, 1, 16, 8, false, true>>(stream, (half*)out, (float*)src, w);
    case 8: return run<&RunStoreQuant<int16_t, int32_t, true, 2, 2, 2, 16, 16, false, false>>(stream, (int16_t*)out, (int32_t*)src, w);
    case 9: return run<&RunStoreQuant<int8_t, int32_t, true, 1, 2, 1, 16, 32, true, true>>(stream, (int8_t*)out, (int32_t*)src, w);
    case 10: return run<&RunStoreQuant<half, float, false, 1, 1, 1, 16, 16, true, false>>(stream, (half*)out, (float*)src, w);
    default: return -1;
    }
}

extern "C" int pto_store_quant_status() { return pto::amd::device_status(); }
