// TEST INFRASTRUCTURE ONLY — never linked into or loaded by the product path.
//
// Thin extern "C" driver over the *unmodified* reference CPU simulator headers
// (/root/reference/include, -D__CPU_SIM -D__PTO_AUTO__).  It is compiled by
// oracle/Makefile into oracle/_ref/libptoref.so and is used for two things only:
//   * validating the plain-C restatement in oracle/pto_oracle.c bit for bit, and
//   * writing the golden fixtures under tests/golden/ (tests/golden/gen_golden.py).
// Every entry point drives the reference's own instruction templates
// (TLOAD / TMOV / TMATMUL[_ACC] / TMATMUL_MX / TSTORE / TQUANT / TDEQUANT) on caller
// buffers; nothing here re-implements arithmetic.
//
// Tiles use the largest static shape the entry point supports with DYNAMIC valid
// rows/cols, so one instantiation serves every (m, k, n) up to that bound.
#include <cstdint>
#include <cstring>
#include <pto/pto-inst.hpp>
#include <pto/common/constants.hpp>

using namespace pto;

namespace {

constexpr int TM = 256;  // max rows of A / C handled by one call
constexpr int TK = 512;  // max contraction length of one TMATMUL (longer K is walked in slabs)
constexpr int TN = 256;  // max cols of B / C handled by one call

using DynShape = Shape<1, 1, 1, DYNAMIC, DYNAMIC>;
using DynStride = Stride<1, 1, 1, DYNAMIC, DYNAMIC>;

template <typename T, Layout L = Layout::ND>
using G2D = GlobalTensor<T, DynShape, DynStride, L>;

template <typename T>
G2D<T, Layout::ND> MakeND(T* p, int rows, int cols, int ld)
{
    return G2D<T, Layout::ND>(p, DynShape(rows, cols), DynStride(ld, 1));
}
template <typename T>
G2D<T, Layout::DN> MakeDN(T* p, int rows, int cols, int ld)
{
    // logical [rows, cols], element (r, c) at p[c * ld + r]
    return G2D<T, Layout::DN>(p, DynShape(rows, cols), DynStride(1, ld));
}

// One-shot or K-split GEMM through TLOAD -> TMOV -> TMATMUL(_ACC) -> TSTORE.
// b_dn != 0: B is stored column-major (element (k, n) at b[n * ldb + k]).
template <typename OutT, typename InT, typename AccT>
int RunGemm(OutT* out, InT* a, InT* b, const AccT* cin, int m, int k, int n, int lda, int ldb, int ldc, int b_dn,
            int kstep, int relu)
{
    if (m < 1 || m > TM || k < 1 || n < 1 || n > TN)
        return -1;
    if (kstep <= 0 || kstep > k)
        kstep = k;
    if (kstep > TK)  // any K, walked in slabs of at most TK through TMATMUL_ACC
        return -1;
    using MatA = Tile<TileType::Mat, InT, TM, TK, BLayout::ColMajor, DYNAMIC, DYNAMIC, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, InT, TK, TN, BLayout::ColMajor, DYNAMIC, DYNAMIC, SLayout::RowMajor, 512>;
    using MatBzn = Tile<TileType::Mat, InT, TK, TN, BLayout::RowMajor, DYNAMIC, DYNAMIC, SLayout::ColMajor, 512>;
    using LeftT = TileLeft<InT, TM, TK, DYNAMIC, DYNAMIC>;
    using RightT = TileRight<InT, TK, TN, DYNAMIC, DYNAMIC>;
    using AccTile = TileAcc<AccT, TM, TN, DYNAMIC, DYNAMIC>;

    AccTile c(m, n);
    bool first = true;
    if (cin != nullptr) {
        for (int i = 0; i < m; ++i)
            for (int j = 0; j < n; ++j)
                c.SetElement(i, j, cin[(size_t)i * ldc + j]);
        first = false;
    }
    for (int k0 = 0; k0 < k; k0 += kstep) {
        const int kc = (k0 + kstep <= k) ? kstep : (k - k0);
        MatA am(m, kc);
        LeftT al(m, kc);
        RightT br(kc, n);
        auto ga = MakeND<InT>(a + k0, m, kc, lda);
        TLOAD(am, ga);
        TMOV(al, am);
        if (b_dn) {
            MatBzn bm(kc, n);
            auto gb = MakeDN<InT>(b + k0, kc, n, ldb);
            TLOAD(bm, gb);
            TMOV(br, bm);
        } else {
            MatB bm(kc, n);
            auto gb = MakeND<InT>(b + (size_t)k0 * ldb, kc, n, ldb);
            TLOAD(bm, gb);
            TMOV(br, bm);
        }
        if (first) {
            TMATMUL(c, al, br);
            first = false;
        } else {
            TMATMUL_ACC(c, c, al, br);
        }
    }
    auto gc = MakeND<OutT>(out, m, n, ldc);
    if (relu)
        TSTORE<AccTile, decltype(gc), AtomicType::AtomicNone, ReluPreMode::NormalRelu>(gc, c);
    else
        TSTORE(gc, c);
    return 0;
}

// scale layouts: 0 = ZZ/NN (fractal), 1 = ND, 2 = DN
template <typename ET, int fmtA>
auto MakeScaleA(float8_e8m0_t* p, int m, int kg)
{
    constexpr Layout L = fmtA == 0 ? Layout::MX_A_ZZ : (fmtA == 1 ? Layout::MX_A_ND : Layout::MX_A_DN);
    using S = TileShape2D<ET, DYNAMIC, DYNAMIC, L>;
    using B = BaseShape2D<ET, DYNAMIC, DYNAMIC, L>;
    return GlobalTensor<ET, S, B, L>(p, S(m, kg), B(m, kg));
}
template <typename ET, int fmtB>
auto MakeScaleB(float8_e8m0_t* p, int kg, int n)
{
    constexpr Layout L = fmtB == 0 ? Layout::MX_B_NN : (fmtB == 1 ? Layout::MX_B_ND : Layout::MX_B_DN);
    using S = TileShape2D<ET, DYNAMIC, DYNAMIC, L>;
    using B = BaseShape2D<ET, DYNAMIC, DYNAMIC, L>;
    return GlobalTensor<ET, S, B, L>(p, S(kg, n), B(kg, n));
}

template <typename InT, int fmt>
int RunGemmMx(float* out, InT* a, InT* b, float8_e8m0_t* sa, float8_e8m0_t* sb, const float* cin, int m, int k, int n,
              int b_dn)
{
    if (m < 1 || m > TM || k < 1 || k > TK || n < 1 || n > TN || (k % 64) != 0)
        return -1;
    if (fmt == 0 && ((m % 16) != 0 || (n % 16) != 0))
        return -2;
    const int kg = k / 32;
    using ET = float8_e8m0_t;
    using MatA = Tile<TileType::Mat, InT, TM, TK, BLayout::ColMajor, DYNAMIC, DYNAMIC, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, InT, TK, TN, BLayout::ColMajor, DYNAMIC, DYNAMIC, SLayout::RowMajor, 512>;
    using MatBzn = Tile<TileType::Mat, InT, TK, TN, BLayout::RowMajor, DYNAMIC, DYNAMIC, SLayout::ColMajor, 512>;
    using MatSA = Tile<TileType::Mat, ET, TM, TK / 32, BLayout::RowMajor, DYNAMIC, DYNAMIC, SLayout::RowMajor, 32>;
    using MatSB = Tile<TileType::Mat, ET, TK / 32, TN, BLayout::ColMajor, DYNAMIC, DYNAMIC, SLayout::ColMajor, 32>;
    using LeftT = TileLeft<InT, TM, TK, DYNAMIC, DYNAMIC>;
    using RightT = TileRight<InT, TK, TN, DYNAMIC, DYNAMIC>;
    using LeftS = TileLeftScale<ET, TM, TK / 32, DYNAMIC, DYNAMIC>;
    using RightS = TileRightScale<ET, TK / 32, TN, DYNAMIC, DYNAMIC>;
    using AccTile = TileAcc<float, TM, TN, DYNAMIC, DYNAMIC>;

    MatA am(m, k);
    LeftT al(m, k);
    RightT br(k, n);
    MatSA sam(m, kg);
    MatSB sbm(kg, n);
    LeftS sal(m, kg);
    RightS sbr(kg, n);
    AccTile c(m, n);

    auto ga = MakeND<InT>(a, m, k, k);
    TLOAD(am, ga);
    TMOV(al, am);
    if (b_dn) {
        MatBzn bm(k, n);
        auto gb = MakeDN<InT>(b, k, n, k);
        TLOAD(bm, gb);
        TMOV(br, bm);
    } else {
        MatB bm(k, n);
        auto gb = MakeND<InT>(b, k, n, n);
        TLOAD(bm, gb);
        TMOV(br, bm);
    }
    auto gsa = MakeScaleA<ET, fmt>(sa, m, kg);
    auto gsb = MakeScaleB<ET, fmt>(sb, kg, n);
    TLOAD<MatSA, decltype(gsa)>(sam, gsa);
    TLOAD<MatSB, decltype(gsb)>(sbm, gsb);
    TMOV(sal, sam);
    TMOV(sbr, sbm);
    if (cin != nullptr) {
        for (int i = 0; i < m; ++i)
            for (int j = 0; j < n; ++j)
                c.SetElement(i, j, cin[(size_t)i * n + j]);
        TMATMUL_MX(c, c, al, sal, br, sbr);
    } else {
        TMATMUL_MX(c, al, sal, br, sbr);
    }
    auto gc = MakeND<float>(out, m, n, n);
    TSTORE(gc, c);
    return 0;
}

// ---- TSTORE with the fix-pipe requantisation (scalar word or per-column fp tile) -------------
template <typename OutT, typename AccT, bool relu>
int RunStoreQuant(OutT* out, const AccT* acc, int m, int n, const uint64_t* scalars, int per_column)
{
    if (m < 1 || m > TM || n < 1 || n > TN)
        return -1;
    using AccTile = TileAcc<AccT, TM, TN, DYNAMIC, DYNAMIC>;
    using FpTile = Tile<TileType::Scaling, uint64_t, 1, TN, BLayout::RowMajor, DYNAMIC, DYNAMIC, SLayout::NoneBox>;
    AccTile c(m, n);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j)
            c.SetElement(i, j, acc[(size_t)i * n + j]);
    auto gc = MakeND<OutT>(out, m, n, n);
    constexpr ReluPreMode rm = relu ? ReluPreMode::NormalRelu : ReluPreMode::NoRelu;
    if (per_column) {
        FpTile fp(1, n);
        for (int j = 0; j < n; ++j)
            fp.SetElement(0, j, scalars[j]);
        TSTORE<AccTile, decltype(gc), FpTile, AtomicType::AtomicNone, rm>(gc, c, fp);
    } else {
        TSTORE<AccTile, decltype(gc), AtomicType::AtomicNone, rm>(gc, c, scalars[0]);
    }
    return 0;
}

// ---- TQUANT / TDEQUANT ----------------------------------------------------------------------
template <int R, int C, bool asym>
int RunQuantInt8(uint8_t* dst, const float* src, const float* scale, const float* offset)
{
    using SrcTile = Tile<TileType::Vec, float, R, C>;
    using DstTile = Tile<TileType::Vec, std::conditional_t<asym, uint8_t, int8_t>, R, C>;
    using ParaTile = Tile<TileType::Vec, float, (R + 7) / 8 * 8, 1, BLayout::ColMajor, R, 1>;
    SrcTile s;
    DstTile d;
    ParaTile sc, off;
    for (int r = 0; r < R; ++r) {
        sc.SetElement(r, 0, scale[r]);
        off.SetElement(r, 0, offset ? offset[r] : 0.0f);
        for (int c = 0; c < C; ++c)
            s.SetElement(r, c, src[r * C + c]);
    }
    if constexpr (asym)
        TQUANT<QuantType::INT8_ASYM>(d, s, sc, &off);
    else
        TQUANT<QuantType::INT8_SYM>(d, s, sc);
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            dst[r * C + c] = (uint8_t)d.GetElement(r, c);
    return 0;
}

// axis = 1: 32-element groups run along a row (ND); axis = 0: along a column (DN).
// dst receives one byte per element for MXFP8 and packed nibbles (row-major, low nibble = even col) for MXFP4.
template <int R, int C, int axis, MxQuantAlg alg, typename SrcT>
int RunQuantMxImpl(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const float* src)
{
    constexpr bool fp4 = (alg == MxQuantAlg::OcpMxFp4E2M1 || alg == MxQuantAlg::NvMxFp4E2M1);
    constexpr int ER = axis == 1 ? R : R / 32;
    constexpr int EC = axis == 1 ? C / 32 : C;
    constexpr int G = ER * EC;
    using SrcTile = Tile<TileType::Vec, SrcT, R, C>;
    using DstTile = Tile<TileType::Vec, std::conditional_t<fp4, float4_e2m1x2_t, int8_t>, R, C>;
    using ExpTile = Tile<TileType::Vec, uint8_t, ER, (EC + 31) / 32 * 32, BLayout::RowMajor, ER, EC>;
    using FlatTile = Tile<TileType::Vec, float, 1, (G + 7) / 8 * 8>;
    SrcTile s;
    DstTile d;
    ExpTile e;
    FlatTile m, sc;
    // The reference clears Rows*Cols bytes of a packed fp4 destination (cpu/TQuant.hpp:451-459), twice what the
    // lazily allocated tile storage holds, so the destination is bound to the simulated UB region instead.
    TASSIGN(d, 0x0);
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            s.SetElement(r, c, static_cast<SrcT>(src[r * C + c]));
    TQUANT<axis, alg, DstTile, SrcTile, ExpTile, FlatTile, FlatTile>(d, s, &e, &m, &sc);
    if constexpr (fp4) {
        std::memcpy(dst, d.data(), R * C / 2);
    } else {
        for (int r = 0; r < R; ++r)
            for (int c = 0; c < C; ++c)
                dst[r * C + c] = (uint8_t)d.GetElement(r, c);
    }
    for (int r = 0; r < ER; ++r)
        for (int c = 0; c < EC; ++c)
            exp[r * EC + c] = e.GetElement(r, c);
    for (int g = 0; g < G; ++g) {
        mx[g] = m.data()[g];
        scaling[g] = sc.data()[g];
    }
    return 0;
}

template <int R, int C, int axis, MxQuantAlg alg, typename SrcT>
int RunQuantMx(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const float* src)
{
    constexpr bool fp4 = (alg == MxQuantAlg::OcpMxFp4E2M1 || alg == MxQuantAlg::NvMxFp4E2M1);
    if constexpr (fp4 && (C % 64) != 0) {
        return -2;  // packed fp4 rows must be 32-byte aligned in the reference tile type
    } else {
        return RunQuantMxImpl<R, C, axis, alg, SrcT>(dst, exp, mx, scaling, src);
    }
}

template <int R, int C, typename SrcT>
int RunDequant(float* dst, const SrcT* src, const float* scale, const float* offset)
{
    using SrcTile = Tile<TileType::Vec, SrcT, R, C>;
    using DstTile = Tile<TileType::Vec, float, R, C>;
    using ParaTile = Tile<TileType::Vec, float, (R + 7) / 8 * 8, 1, BLayout::ColMajor, R, 1>;
    SrcTile s;
    DstTile d;
    ParaTile sc, off;
    for (int r = 0; r < R; ++r) {
        sc.SetElement(r, 0, scale[r]);
        off.SetElement(r, 0, offset[r]);
        for (int c = 0; c < C; ++c)
            s.SetElement(r, c, src[r * C + c]);
    }
    TDEQUANT(d, s, sc, off);
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            dst[r * C + c] = d.GetElement(r, c);
    return 0;
}

// Parameter tiles as the reference reads them: TDEQUANT clamps the parameter column to the tile's valid columns
// (TDeQuant.hpp:24-30); TQUANT INT8 reads column 0 and clamps the row to the valid rows (GetParamValue, TQuant.hpp:78-84).
template <int PC>
int RunDequantPara(float* dst, const int8_t* src, const float* scale, const float* offset)
{
    constexpr int R = 16, C = 64;
    using SrcTile = Tile<TileType::Vec, int8_t, R, C>;
    using DstTile = Tile<TileType::Vec, float, R, C>;
    using ParaTile = Tile<TileType::Vec, float, R, 8, BLayout::RowMajor, R, PC>;
    SrcTile s;
    DstTile d;
    ParaTile sc, off;
    for (int r = 0; r < R; ++r) {
        for (int c = 0; c < PC; ++c) {
            sc.SetElement(r, c, scale[r * PC + c]);
            off.SetElement(r, c, offset[r * PC + c]);
        }
        for (int c = 0; c < C; ++c)
            s.SetElement(r, c, src[r * C + c]);
    }
    TDEQUANT(d, s, sc, off);
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            dst[r * C + c] = d.GetElement(r, c);
    return 0;
}

template <int PR, bool asym>
int RunQuantInt8Para(uint8_t* dst, const float* src, const float* scale, const float* offset)
{
    constexpr int R = 16, C = 64;
    using SrcTile = Tile<TileType::Vec, float, R, C>;
    using DstTile = Tile<TileType::Vec, std::conditional_t<asym, uint8_t, int8_t>, R, C>;
    using ParaTile = Tile<TileType::Vec, float, R, 8, BLayout::RowMajor, PR, 3>;
    SrcTile s;
    DstTile d;
    ParaTile sc, off;
    for (int r = 0; r < PR; ++r)
        for (int c = 0; c < 3; ++c) {  // columns 1 and 2 hold other values: only column 0 may be read
            sc.SetElement(r, c, c == 0 ? scale[r] : -1000.0f);
            off.SetElement(r, c, c == 0 ? offset[r] : 999.0f);
        }
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            s.SetElement(r, c, src[r * C + c]);
    if constexpr (asym)
        TQUANT<QuantType::INT8_ASYM>(d, s, sc, &off);
    else
        TQUANT<QuantType::INT8_SYM>(d, s, sc);
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            dst[r * C + c] = (uint8_t)d.GetElement(r, c);
    return 0;
}

template <typename TileT>
int64_t TileOffset(int r, int c)
{
    return (int64_t)GetTileElementOffset<TileT>(r, c);
}

}  // namespace

extern "C" {

void ref_init(int arch_a5)
{
    NPU_MEMORY_INIT(arch_a5 ? NPUArch::A5 : NPUArch::A2A3);
}

int ref_gemm_f16(float* out, const uint16_t* a, const uint16_t* b, const float* cin, int m, int k, int n, int b_dn,
                 int kstep)
{
    return RunGemm<float, half, float>(out, (half*)a, (half*)b, cin, m, k, n, k, b_dn ? k : n, n, b_dn, kstep, 0);
}
int ref_gemm_f16_out_f16(uint16_t* out, const uint16_t* a, const uint16_t* b, int m, int k, int n, int b_dn, int kstep,
                         int relu)
{
    return RunGemm<half, half, float>((half*)out, (half*)a, (half*)b, nullptr, m, k, n, k, b_dn ? k : n, n, b_dn,
                                      kstep, relu);
}
int ref_gemm_f32(float* out, const float* a, const float* b, const float* cin, int m, int k, int n, int b_dn, int kstep)
{
    return RunGemm<float, float, float>(out, (float*)a, (float*)b, cin, m, k, n, k, b_dn ? k : n, n, b_dn, kstep, 0);
}
int ref_gemm_i8(int32_t* out, const int8_t* a, const int8_t* b, const int32_t* cin, int m, int k, int n, int b_dn,
                int kstep)
{
    return RunGemm<int32_t, int8_t, int32_t>(out, (int8_t*)a, (int8_t*)b, cin, m, k, n, k, b_dn ? k : n, n, b_dn,
                                             kstep, 0);
}
int ref_gemm_e4m3(float* out, const uint8_t* a, const uint8_t* b, const float* cin, int m, int k, int n, int b_dn,
                  int kstep)
{
    return RunGemm<float, float8_e4m3_t, float>(out, (float8_e4m3_t*)a, (float8_e4m3_t*)b, cin, m, k, n, k,
                                                b_dn ? k : n, n, b_dn, kstep, 0);
}
int ref_gemm_e5m2(float* out, const uint8_t* a, const uint8_t* b, const float* cin, int m, int k, int n, int b_dn,
                  int kstep)
{
    return RunGemm<float, float8_e5m2_t, float>(out, (float8_e5m2_t*)a, (float8_e5m2_t*)b, cin, m, k, n, k,
                                                b_dn ? k : n, n, b_dn, kstep, 0);
}

// dtype: 0 = e4m3, 1 = e5m2, 2 = e2m1x2 (packed), 3 = e1m2x2 (packed); scale_fmt: 0 ZZ/NN, 1 ND/ND, 2 DN/DN
int ref_gemm_mx(float* out, const uint8_t* a, const uint8_t* b, const uint8_t* sa, const uint8_t* sb, const float* cin,
                int m, int k, int n, int dtype, int scale_fmt, int b_dn)
{
    auto* psa = (float8_e8m0_t*)sa;
    auto* psb = (float8_e8m0_t*)sb;
#define PTO_REF_MX(T)                                                                   \
    switch (scale_fmt) {                                                                \
        case 0:                                                                         \
            return RunGemmMx<T, 0>(out, (T*)a, (T*)b, psa, psb, cin, m, k, n, b_dn);    \
        case 1:                                                                         \
            return RunGemmMx<T, 1>(out, (T*)a, (T*)b, psa, psb, cin, m, k, n, b_dn);    \
        case 2:                                                                         \
            return RunGemmMx<T, 2>(out, (T*)a, (T*)b, psa, psb, cin, m, k, n, b_dn);    \
        default:                                                                        \
            return -9;                                                                  \
    }
    switch (dtype) {
        case 0:
            PTO_REF_MX(float8_e4m3_t)
        case 1:
            PTO_REF_MX(float8_e5m2_t)
        case 2:
            PTO_REF_MX(float4_e2m1x2_t)
        case 3:
            PTO_REF_MX(float4_e1m2x2_t)
        default:
            return -9;
    }
#undef PTO_REF_MX
}


// ---- fix-pipe requantising stores -----------------------------------------------------------
int ref_store_f32_i8(int8_t* out, const float* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<int8_t, float, true>(out, acc, m, n, q, per_col) :
                  RunStoreQuant<int8_t, float, false>(out, acc, m, n, q, per_col);
}
int ref_store_f32_u8(uint8_t* out, const float* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<uint8_t, float, true>(out, acc, m, n, q, per_col) :
                  RunStoreQuant<uint8_t, float, false>(out, acc, m, n, q, per_col);
}
int ref_store_f32_f16(uint16_t* out, const float* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<half, float, true>((half*)out, acc, m, n, q, per_col) :
                  RunStoreQuant<half, float, false>((half*)out, acc, m, n, q, per_col);
}
int ref_store_i32_i8(int8_t* out, const int32_t* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<int8_t, int32_t, true>(out, acc, m, n, q, per_col) :
                  RunStoreQuant<int8_t, int32_t, false>(out, acc, m, n, q, per_col);
}
int ref_store_i32_f16(uint16_t* out, const int32_t* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<half, int32_t, true>((half*)out, acc, m, n, q, per_col) :
                  RunStoreQuant<half, int32_t, false>((half*)out, acc, m, n, q, per_col);
}

int ref_store_i32_i16(int16_t* out, const int32_t* acc, int m, int n, const uint64_t* q, int per_col, int relu)
{
    return relu ? RunStoreQuant<int16_t, int32_t, true>(out, acc, m, n, q, per_col) :
                  RunStoreQuant<int16_t, int32_t, false>(out, acc, m, n, q, per_col);
}

// the fix-pipe's control bits as the simulator reads them (get_task_cookie, common/cpu_stub.hpp:606-612); bit 48 is the
// saturate-inf control of quantize_element (cpu/common.hpp:146).  Per calling thread.
void ref_set_task_cookie(uint64_t cookie) { pto::cpu_sim::set_task_cookie(cookie); }

// static_cast<double>(hifloat8_t::FromRaw(code)) for all 256 codes (cpu/Hifloat8.hpp)
void ref_hif8_table(double* out256)
{
    for (int c = 0; c < 256; ++c)
        out256[c] = static_cast<double>(hifloat8_t::FromRaw(static_cast<uint8_t>(c)));
}

// ---- TQUANT / TDEQUANT; shape_id selects one of the compiled static shapes -------------------
// shape ids: 0 = 4x32, 1 = 2x128, 2 = 2x256, 3 = 16x64, 4 = 8x512, 5 = 64x64, 6 = 32x96
#define PTO_REF_SHAPES(X) X(0, 4, 32) X(1, 2, 128) X(2, 2, 256) X(3, 16, 64) X(4, 8, 512) X(5, 64, 64) X(6, 32, 96)

int ref_shape(int id, int* rows, int* cols)
{
#define X(i, r, c)   \
    if (id == i) {   \
        *rows = r;   \
        *cols = c;   \
        return 0;    \
    }
    PTO_REF_SHAPES(X)
#undef X
    return -1;
}

int ref_tquant_int8(int shape_id, int asym, uint8_t* dst, const float* src, const float* scale, const float* offset)
{
#define X(i, r, c)                                                            \
    if (shape_id == i)                                                        \
        return asym ? RunQuantInt8<r, c, true>(dst, src, scale, offset) :     \
                      RunQuantInt8<r, c, false>(dst, src, scale, offset);
    PTO_REF_SHAPES(X)
#undef X
    return -1;
}

// alg: 0 OCP-FP8, 1 NV-FP8, 2 OCP-FP4, 3 NV-FP4; axis 1 = groups along rows' K (ND), 0 = along columns (DN)
// src_f16 != 0: the source tile is half precision (values are narrowed to fp16 first)
int ref_tquant_mx(int shape_id, int alg, int axis, int src_f16, uint8_t* dst, uint8_t* exp, float* mx, float* scaling,
                  const float* src)
{
#define Y(r, c, ax, A)                                                         \
    return src_f16 ? RunQuantMx<r, c, ax, A, half>(dst, exp, mx, scaling, src) : \
                     RunQuantMx<r, c, ax, A, float>(dst, exp, mx, scaling, src);
#define Z(r, c, ax)                                  \
    switch (alg) {                                   \
        case 0:                                      \
            Y(r, c, ax, MxQuantAlg::OcpMxFp8E4M3)    \
        case 1:                                      \
            Y(r, c, ax, MxQuantAlg::NvMxFp8E4M3)     \
        case 2:                                      \
            Y(r, c, ax, MxQuantAlg::OcpMxFp4E2M1)    \
        case 3:                                      \
            Y(r, c, ax, MxQuantAlg::NvMxFp4E2M1)     \
        default:                                     \
            return -9;                               \
    }
    if (axis == 1) {
        if (shape_id == 0) { Z(4, 32, 1) }
        if (shape_id == 1) { Z(2, 128, 1) }
        if (shape_id == 2) { Z(2, 256, 1) }
        if (shape_id == 3) { Z(16, 64, 1) }
        if (shape_id == 4) { Z(8, 512, 1) }
        if (shape_id == 5) { Z(64, 64, 1) }
        if (shape_id == 6) { Z(32, 96, 1) }
    } else {
        if (shape_id == 5) { Z(64, 64, 0) }
        if (shape_id == 6) { Z(32, 96, 0) }
    }
#undef Z
#undef Y
    return -1;
}

int ref_tdequant(int shape_id, int src_kind, float* dst, const void* src, const float* scale, const float* offset)
{
#define X(i, r, c)                                                                         \
    if (shape_id == i) {                                                                   \
        if (src_kind == 0)                                                                 \
            return RunDequant<r, c, int8_t>(dst, (const int8_t*)src, scale, offset);       \
        if (src_kind == 1)                                                                 \
            return RunDequant<r, c, int16_t>(dst, (const int16_t*)src, scale, offset);     \
        return RunDequant<r, c, int32_t>(dst, (const int32_t*)src, scale, offset);         \
    }
    PTO_REF_SHAPES(X)
#undef X
    return -1;
}

// 16 x 64 int8 source; scale / offset [16][para_cols], para_cols 1, 3 or 8
int ref_tdequant_para(int para_cols, float* dst, const int8_t* src, const float* scale, const float* offset)
{
    switch (para_cols) {
        case 1: return RunDequantPara<1>(dst, src, scale, offset);
        case 3: return RunDequantPara<3>(dst, src, scale, offset);
        case 8: return RunDequantPara<8>(dst, src, scale, offset);
        default: return -1;
    }
}

// 16 x 64 f32 source; scale / offset [para_rows], para_rows 1, 5 or 16
int ref_tquant_int8_para(int para_rows, int asym, uint8_t* dst, const float* src, const float* scale, const float* offset)
{
#define P(n)                                                                         \
    if (para_rows == n)                                                              \
        return asym ? RunQuantInt8Para<n, true>(dst, src, scale, offset) :           \
                      RunQuantInt8Para<n, false>(dst, src, scale, offset);
    P(1) P(5) P(16)
#undef P
    return -1;
}

// ---- scalar helpers --------------------------------------------------------------------------
// type: 0 e4m3, 1 e5m2, 2 e2m1, 3 e1m2, 4 e8m0
double ref_mx_decode(int type, unsigned raw)
{
    switch (type) {
        case 0: return (double)float8_e4m3_t::FromRaw((uint8_t)raw);
        case 1: return (double)float8_e5m2_t::FromRaw((uint8_t)raw);
        case 2: return (double)float4_e2m1x2_t::FromRaw((uint8_t)raw);
        case 3: return (double)float4_e1m2x2_t::FromRaw((uint8_t)raw);
        default: return (double)float8_e8m0_t::FromRaw((uint8_t)raw);
    }
}
unsigned ref_mx_encode_trunc(int type, double v)
{
    switch (type) {
        case 0: return float8_e4m3_t(v).RawData();
        case 1: return float8_e5m2_t(v).RawData();
        case 2: return float4_e2m1x2_t(v).RawData();
        case 3: return float4_e1m2x2_t(v).RawData();
        default: return float8_e8m0_t(v).RawData();
    }
}
unsigned ref_mx_encode_round(int type, double v, int round_mode, int sat_on)
{
    const auto rm = static_cast<RoundMode>(round_mode);
    const auto sm = sat_on ? SaturationMode::ON : SaturationMode::OFF;
    switch (type) {
        case 0: return float8_e4m3_t(v, rm, sm).RawData();
        case 1: return float8_e5m2_t(v, rm, sm).RawData();
        case 2: return float4_e2m1x2_t(v, rm).RawData();
        default: return float4_e1m2x2_t(v, rm).RawData();
    }
}
unsigned ref_encode_e4m3fn(float v, int nv) { return nv ? cpu_quant::EncodeE4M3Fn<QuantScaleAlg::NV>(v) : cpu_quant::EncodeE4M3Fn<QuantScaleAlg::OCP>(v); }
unsigned ref_encode_e2m1_magic(float v) { return cpu_quant::EncodeE2M1Magic(v); }
// which: 0 OCP-FP8, 1 NV-FP8, 2 OCP-FP4, 3 NV-FP4
unsigned ref_shared_exponent(int which, float maxabs)
{
    switch (which) {
        case 0: return cpu_quant::ComputeMxSharedExponent<QuantType::MXFP8, QuantScaleAlg::OCP>(maxabs);
        case 1: return cpu_quant::ComputeMxSharedExponent<QuantType::MXFP8, QuantScaleAlg::NV>(maxabs);
        case 2: return cpu_quant::ComputeMxSharedExponent<QuantType::MXFP4_E2M1, QuantScaleAlg::OCP>(maxabs);
        default: return cpu_quant::ComputeMxSharedExponent<QuantType::MXFP4_E2M1, QuantScaleAlg::NV>(maxabs);
    }
}
float ref_group_scaling(int which, float maxabs, unsigned e8m0)
{
    switch (which) {
        case 0: return cpu_quant::ComputeMxGroupScaling<QuantType::MXFP8, QuantScaleAlg::OCP>(maxabs, (uint8_t)e8m0);
        case 1: return cpu_quant::ComputeMxGroupScaling<QuantType::MXFP8, QuantScaleAlg::NV>(maxabs, (uint8_t)e8m0);
        case 2: return cpu_quant::ComputeMxGroupScaling<QuantType::MXFP4_E2M1, QuantScaleAlg::OCP>(maxabs, (uint8_t)e8m0);
        default: return cpu_quant::ComputeMxGroupScaling<QuantType::MXFP4_E2M1, QuantScaleAlg::NV>(maxabs, (uint8_t)e8m0);
    }
}
float ref_extract_m1(uint64_t word, int vector_mode)
{
    return vector_mode ? extract_m1_from_quant<true>(word) : extract_m1_from_quant<false>(word);
}

// Tile element offsets for the layouts the hot path touches (tile static shape 64 x 128, or 64 x 8 / 8 x 64 for
// the scale tiles).  kind: 0 Mat-NZ f16, 1 Mat-ZN f16, 2 Left f16, 3 Right f16, 4 Acc f32, 5 Mat-NZ i8,
// 6 Mat-NZ fp4, 7 LeftScale, 8 RightScale, 9 Vec row-major f32, 10 Vec col-major f32, 11 Mat-NZ f32
int64_t ref_tile_offset(int kind, int r, int c)
{
    switch (kind) {
        case 0: return TileOffset<Tile<TileType::Mat, half, 64, 128, BLayout::ColMajor, 64, 128, SLayout::RowMajor, 512>>(r, c);
        case 1: return TileOffset<Tile<TileType::Mat, half, 64, 128, BLayout::RowMajor, 64, 128, SLayout::ColMajor, 512>>(r, c);
        case 2: return TileOffset<TileLeft<half, 64, 128>>(r, c);
        case 3: return TileOffset<TileRight<half, 64, 128>>(r, c);
        case 4: return TileOffset<TileAcc<float, 64, 128>>(r, c);
        case 5: return TileOffset<Tile<TileType::Mat, int8_t, 64, 128, BLayout::ColMajor, 64, 128, SLayout::RowMajor, 512>>(r, c);
        case 6: return TileOffset<Tile<TileType::Mat, float4_e2m1x2_t, 64, 128, BLayout::ColMajor, 64, 128, SLayout::RowMajor, 512>>(r, c);
        case 7: return TileOffset<TileLeftScale<float8_e8m0_t, 64, 8>>(r, c);
        case 8: return TileOffset<TileRightScale<float8_e8m0_t, 8, 64>>(r, c);
        case 9: return TileOffset<Tile<TileType::Vec, float, 64, 128>>(r, c);
        case 10: return TileOffset<Tile<TileType::Vec, float, 64, 128, BLayout::ColMajor>>(r, c);
        case 11: return TileOffset<Tile<TileType::Mat, float, 64, 128, BLayout::ColMajor, 64, 128, SLayout::RowMajor, 512>>(r, c);
        default: return -1;
    }
}

// Global (GM) element offset of logical (r, c) for the MX scale layouts, rows x cols logical extent.
// layout: 0 MX_A_ZZ, 1 MX_A_ND, 2 MX_A_DN, 3 MX_B_NN, 4 MX_B_ND, 5 MX_B_DN
int64_t ref_mx_scale_offset(int layout, int rows, int cols, int r, int c)
{
    using ET = float8_e8m0_t;
#define W(L)                                                                                                 \
    {                                                                                                        \
        using S = TileShape2D<ET, DYNAMIC, DYNAMIC, L>;                                                      \
        using B = BaseShape2D<ET, DYNAMIC, DYNAMIC, L>;                                                      \
        GlobalTensor<ET, S, B, L> g(nullptr, S(rows, cols), B(rows, cols));                                  \
        std::vector<int64_t> sh, st;                                                                         \
        for (int d = 0; d < 5; ++d) {                                                                        \
            sh.push_back(g.GetShape(d));                                                                     \
            st.push_back(g.GetStride(d));                                                                    \
        }                                                                                                    \
        return (int64_t)MapTileIndicesToGlobalOffset<decltype(g)>(r, c, sh, st);                             \
    }
    switch (layout) {
        case 0: W(Layout::MX_A_ZZ)
        case 1: W(Layout::MX_A_ND)
        case 2: W(Layout::MX_A_DN)
        case 3: W(Layout::MX_B_NN)
        case 4: W(Layout::MX_B_ND)
        case 5: W(Layout::MX_B_DN)
        default: return -1;
    }
#undef W
}

// GM element offset of logical (r, c) of a 5-D GlobalTensor with static shape and padded strides.
// which: 0 ND Shape<2,3,4,8,16>, 1 DN Shape<2,3,4,8,16>, 2 NZ Shape<1,4,3,16,8> (the three global layouts TLOAD takes
// for matrix operands).  shape_out / stride_out receive what the tensor reports.  Logical extents as the
// simulator's TLOAD walks them (cpu/TLoad.hpp): ND rows = s0*s1*s2*s3, cols = s4; DN rows = s3,
// cols = s0*s1*s2*s4; NZ rows = s2*s3, cols = s0*s1*s4.
int64_t ref_global_offset(int which, int r, int c, int64_t* shape_out, int64_t* stride_out)
{
#define G(L, SH, ST)                                                                                         \
    {                                                                                                        \
        GlobalTensor<float, SH, ST, L> g(nullptr);                                                           \
        std::vector<int64_t> sh, st;                                                                         \
        for (int d = 0; d < 5; ++d) {                                                                        \
            sh.push_back(g.GetShape(d));                                                                     \
            st.push_back(g.GetStride(d));                                                                    \
            if (shape_out) shape_out[d] = sh[d];                                                             \
            if (stride_out) stride_out[d] = st[d];                                                           \
        }                                                                                                    \
        return (int64_t)MapTileIndicesToGlobalOffset<decltype(g)>(r, c, sh, st);                             \
    }
    using S0 = Shape<2, 3, 4, 8, 16>;
    using S2 = Shape<1, 4, 3, 16, 8>;
    using T0 = Stride<3 * 4 * 8 * 20 + 12, 4 * 8 * 20 + 4, 8 * 20, 20, 1>;   // row pitch 20 > 16, gaps between batches
    using T1 = Stride<3 * 4 * 16 * 10 + 6, 4 * 16 * 10 + 2, 16 * 10, 1, 10>; // column pitch 10 > 8
    using T2 = Stride<4 * 3 * 128 + 64, 3 * 128 + 16, 128, 8, 1>;
    switch (which) {
        case 0: G(Layout::ND, S0, T0)
        case 1: G(Layout::DN, S0, T1)
        case 2: G(Layout::NZ, S2, T2)
        default: return -1;
    }
#undef G
}

// Shape and stride the whole-matrix helpers TileShape2D / BaseShape2D give a [rows, cols] float matrix.
// layout: 0 ND, 1 DN, 2 NZ
int ref_layout_2d(int layout, int rows, int cols, int64_t* shape_out, int64_t* stride_out)
{
#define W(L)                                                                                                 \
    {                                                                                                        \
        using S = TileShape2D<float, DYNAMIC, DYNAMIC, L>;                                                   \
        using B = BaseShape2D<float, DYNAMIC, DYNAMIC, L>;                                                   \
        GlobalTensor<float, S, B, L> g(nullptr, S(rows, cols), B(rows, cols));                               \
        for (int d = 0; d < 5; ++d) {                                                                        \
            shape_out[d] = g.GetShape(d);                                                                    \
            stride_out[d] = g.GetStride(d);                                                                  \
        }                                                                                                    \
        return 0;                                                                                            \
    }
    switch (layout) {
        case 0: W(Layout::ND)
        case 1: W(Layout::DN)
        case 2: W(Layout::NZ)
        default: return -1;
    }
#undef W
}

// TQuant.hpp ReorderExponentZZ on a [rows][group_cols] exponent matrix
void ref_reorder_exp_zz(uint8_t* dst, const uint8_t* exp, int rows, int group_cols)
{
    std::vector<uint8_t> in(exp, exp + (size_t)rows * group_cols);
    auto out = pto::cpu_quant::ReorderExponentZZ(in, rows, group_cols);
    std::copy(out.begin(), out.end(), dst);
}

}  // extern "C"

