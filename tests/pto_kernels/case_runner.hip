// A test main without a test framework, in the shape of the reference's (tests/cpu/st/testcase/tmatmul/main.cpp:40-95,
// tests/cpu/st/testcase/tmatmul_mx/main.cpp:58-148): aclrt* runtime calls, host buffers filled from the reference
// generators' distributions (tmatmul/gen_data.py, tmatmul_mx/gen_data.py), one Launch call, a host-side golden and a
// comparison with the semantics of the reference's ResultCmp (tests/common/test_common.h:231-309).
//
//   case_runner <case>      exit status 0 = match, 1 = mismatch, 2 = usage / runtime error
//   case_runner --data <dir> --manifest <file> [-l] [-t <suite>[.<case>]]...
//                           the reference's own case lists (tmatmul, tmatmul_mx, tstore_acc2gm, tdequant), inputs and
//                           goldens read from <dir>/<suite>/<case>/*.bin, one manifest line per case (written by
//                           tests/golden/gen_runner_cases.py); -l lists the cases, -t selects a suite or one case (the
//                           habit of tests/run_cpu.py -t), no -t runs them all.  Every case runs through the C ABI; a
//                           case whose manifest line names a compiled PTO kernel (k<id>) runs through that as well.
//
// Cases:
//   tmatmul       PTO kernel RunTMATMUL (header layer): f16 40x50x60 -> f32, inputs randint(1, 5)          [tmatmul case1]
//   tmatmul_i8    PTO kernel RunTMATMUL: int8 6x7x8 -> int32                                              [tmatmul case2]
//   tmatmul_mx    PTO kernel RunTMATMULMX: e4m3 127x72x64, scales 127..129 in the ZZ / NN layouts          [tmatmul_mx case2]
//   gemm          C ABI ptoamd_gemm: bf16 256x384x512 -> f32, B column-major
//   gemm_mx       C ABI ptoamd_gemm_mx: e4m3 128x256x512, scales in the plain row layouts
//   quant_gemm    C ABI ptoamd_tquant_mx (OCP MXFP8) of both operands, then ptoamd_gemm_mx on the codes
// The C ABI cases leave one record each in $PTOAMD_TRACE_DIR when that is set.
#include <pto/acl_runtime.hpp>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

extern "C" int pto_kernels_launch(int id, void* out, void* src0, void* src1, void* src2, void* stream);
extern "C" int pto_kernels_status();
extern "C" int pto_store_quant_launch(int id, void* out, void* src, void* words, int saturate, void* stream);
extern "C" int pto_store_quant_status();
extern "C" int pto_boundary_launch_mx(int id, void* out, void* a, void* b, void* sa, void* sb, void* bias, void* stream);
extern "C" int pto_boundary_status();

// ResultCmp: an element is wrong when both its absolute and its relative error exceed eps (or NaN-ness differs); the run
// fails when more than eps * size elements are wrong, or when more than zeroCountThreshold outputs are zero where the
// golden is not.
template <typename T>
static bool ResultCmp(const std::vector<T>& expected, const T* actual, float eps, size_t zeroCountThreshold = 1000)
{
    const size_t threshold = (size_t)(expected.size() * eps);
    float maxDiff = 0, maxDiffRatio = 0;
    size_t zeroCount = 0, errCount = 0;
    for (size_t i = 0; i < expected.size(); ++i) {
        const float e = (float)expected[i], a = (float)actual[i];
        const float diff = std::fabs(e - a), rel = std::fabs(diff / e);
        if (!std::isnan(diff))
            maxDiff = std::fmax(diff, maxDiff);
        if (!std::isnan(rel))
            maxDiffRatio = std::fmax(rel, maxDiffRatio);
        zeroCount += (std::fabs(a) <= 1e-6f && std::fabs(e) > 1e-6f) ? 1 : 0;
        errCount += ((diff > eps && rel > eps) || std::isnan(e) != std::isnan(a)) ? 1 : 0;
    }
    printf("max diff: %g, diff threshold: %g, max diff ratio: %g, err count: %zu, err threshold: %zu, act zero count: %zu\n",
           maxDiff, eps, maxDiffRatio, errCount, threshold, zeroCount);
    return errCount <= threshold && zeroCount <= zeroCountThreshold;
}

#define RT(expr)                                                                  \
    do {                                                                          \
        if ((expr) != 0) {                                                        \
            fprintf(stderr, "%s failed: %s\n", #expr, ptoamd_last_error());       \
            exit(2);                                                              \
        }                                                                         \
    } while (0)

struct DeviceBuffer {
    void* dev = nullptr;
    size_t bytes;
    explicit DeviceBuffer(size_t n) : bytes(n ? n : 16) { RT(aclrtMalloc(&dev, bytes, ACL_MEM_MALLOC_HUGE_FIRST)); }
    DeviceBuffer(const void* host, size_t n) : DeviceBuffer(n) { RT(aclrtMemcpy(dev, bytes, host, n, ACL_MEMCPY_HOST_TO_DEVICE)); }
    ~DeviceBuffer() { aclrtFree(dev); }
    template <typename T>
    std::vector<T> download(size_t count) const
    {
        std::vector<T> h(count);
        RT(aclrtMemcpy(h.data(), count * sizeof(T), dev, count * sizeof(T), ACL_MEMCPY_DEVICE_TO_HOST));
        return h;
    }
};

static uint16_t f16_bits(float v)
{
    const _Float16 h = (_Float16)v;
    uint16_t b;
    memcpy(&b, &h, 2);
    return b;
}
static uint16_t bf16_bits(float v)  // v is chosen bf16-representable
{
    uint32_t b;
    memcpy(&b, &v, 4);
    return (uint16_t)(b >> 16);
}
// E4M3 codes of the integers -10 .. 10 (9 is not representable and becomes 8, as a cast would round it)
static uint8_t e4m3_of_int(int v)
{
    static const uint8_t mag[11] = {0x00, 0x38, 0x40, 0x44, 0x48, 0x4A, 0x4C, 0x4E, 0x50, 0x50, 0x52};
    return (uint8_t)((v < 0 ? 0x80 : 0) | mag[v < 0 ? -v : v]);
}
static float e4m3_value(uint8_t c)
{
    const int e = (c >> 3) & 0xF, m = c & 7;
    const float v = e == 0 ? std::ldexp((float)m, -9) : std::ldexp(1.0f + m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

static bool case_tmatmul(void* stream)
{
    const int m = 40, k = 50, n = 60;
    std::mt19937 rng(19);
    std::uniform_int_distribution<int> d(1, 4);
    std::vector<uint16_t> a(m * k), b(k * n);
    std::vector<float> av(m * k), bv(k * n), golden(m * n);
    for (int i = 0; i < m * k; ++i)
        a[i] = f16_bits(av[i] = (float)d(rng));
    for (int i = 0; i < k * n; ++i)
        b[i] = f16_bits(bv[i] = (float)d(rng));
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (double)av[i * k + kk] * bv[kk * n + j];
            golden[i * n + j] = (float)s;
        }
    DeviceBuffer da(a.data(), a.size() * 2), db(b.data(), b.size() * 2), dc((size_t)m * n * 4);
    RT(pto_kernels_launch(1, dc.dev, da.dev, db.dev, nullptr, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto out = dc.download<float>((size_t)m * n);
    return pto_kernels_status() == 0 && ResultCmp(golden, out.data(), 0.001f);
}

static bool case_tmatmul_i8(void* stream)
{
    const int m = 6, k = 7, n = 8;
    std::mt19937 rng(20);
    std::uniform_int_distribution<int> d(-128, 127);
    std::vector<int8_t> a(m * k), b(k * n);
    std::vector<int32_t> golden(m * n);
    for (auto& v : a)
        v = (int8_t)d(rng);
    for (auto& v : b)
        v = (int8_t)d(rng);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            int32_t s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (int32_t)a[i * k + kk] * b[kk * n + j];
            golden[i * n + j] = s;
        }
    DeviceBuffer da(a.data(), a.size()), db(b.data(), b.size()), dc((size_t)m * n * 4);
    RT(pto_kernels_launch(2, dc.dev, da.dev, db.dev, nullptr, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto out = dc.download<int32_t>((size_t)m * n);
    return pto_kernels_status() == 0 && ResultCmp(golden, out.data(), 0.001f);
}

// scale byte offsets of the boxed layouts (cpu/tile_offsets.hpp:233-268): 16 rows (columns) x 2 K-groups per box
static size_t zz_offset(int r, int g, int groups) { return (size_t)(r / 16) * groups * 16 + (g / 2) * 32 + (r % 16) * 2 + g % 2; }

static bool case_tmatmul_mx(void* stream)
{
    const int m = 127, k = 72, n = 64, mp = 128, kAlign = 128, kg = kAlign / 32;
    std::mt19937 rng(21);
    std::uniform_int_distribution<int> d(-10, 9), ds(127, 129);
    std::vector<uint8_t> a(m * k), b(k * n), sa((size_t)mp * kg, 0), sb((size_t)kg * n, 0);
    std::vector<float> as(m * kg), bs(kg * n), golden(m * n);
    for (auto& v : a)
        v = e4m3_of_int(d(rng));
    for (auto& v : b)
        v = e4m3_of_int(d(rng));
    for (int i = 0; i < m; ++i)
        for (int g = 0; g < kg; ++g) {
            const int e = ds(rng);
            as[i * kg + g] = std::ldexp(1.0f, e - 127);
            sa[zz_offset(i, g, kg)] = (uint8_t)e;
        }
    for (int g = 0; g < kg; ++g)
        for (int j = 0; j < n; ++j) {
            const int e = ds(rng);
            bs[g * n + j] = std::ldexp(1.0f, e - 127);
            sb[zz_offset(j, g, kg)] = (uint8_t)e;  // MX_B_NN is the same boxing with the roles of row and column swapped
        }
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (double)e4m3_value(a[i * k + kk]) * as[i * kg + kk / 32] * e4m3_value(b[kk * n + j]) * bs[(kk / 32) * n + j];
            golden[i * n + j] = (float)s;
        }
    DeviceBuffer da(a.data(), a.size()), db(b.data(), b.size()), dsa(sa.data(), sa.size()), dsb(sb.data(), sb.size()), dc((size_t)m * n * 4);
    RT(pto_boundary_launch_mx(2, dc.dev, da.dev, db.dev, dsa.dev, dsb.dev, nullptr, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto out = dc.download<float>((size_t)m * n);
    return pto_boundary_status() == 0 && ResultCmp(golden, out.data(), 0.001f);
}

static bool case_gemm(void* stream)
{
    const int m = 256, n = 384, k = 512;
    std::mt19937 rng(22);
    std::uniform_int_distribution<int> d(-8, 8);
    std::vector<uint16_t> a((size_t)m * k), b((size_t)n * k);
    std::vector<float> av(a.size()), bv(b.size()), golden((size_t)m * n);
    for (size_t i = 0; i < a.size(); ++i)
        a[i] = bf16_bits(av[i] = d(rng) * 0.125f);
    for (size_t i = 0; i < b.size(); ++i)
        b[i] = bf16_bits(bv[i] = d(rng) * 0.25f);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (double)av[(size_t)i * k + kk] * bv[(size_t)j * k + kk];
            golden[(size_t)i * n + j] = (float)s;
        }
    DeviceBuffer da(a.data(), a.size() * 2), db(b.data(), b.size() * 2), dc((size_t)m * n * 4);
    RT(ptoamd_gemm(dc.dev, PTOAMD_F32, da.dev, db.dev, PTOAMD_BF16, nullptr, m, n, k, k, k, n, PTOAMD_B_DN, 0, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto out = dc.download<float>((size_t)m * n);
    printf("kernel: %s\n", ptoamd_last_kernel());
    return ResultCmp(golden, out.data(), 0.001f);
}

static bool case_gemm_mx(void* stream)
{
    const int m = 128, n = 256, k = 512, kg = k / 32;
    std::mt19937 rng(23);
    std::uniform_int_distribution<int> d(-10, 9), ds(125, 130);
    std::vector<uint8_t> a((size_t)m * k), b((size_t)n * k), sa((size_t)m * kg), sb((size_t)n * kg);
    std::vector<float> golden((size_t)m * n);
    for (auto& v : a)
        v = e4m3_of_int(d(rng));
    for (auto& v : b)
        v = e4m3_of_int(d(rng));
    for (auto& v : sa)
        v = (uint8_t)ds(rng);
    for (auto& v : sb)
        v = (uint8_t)ds(rng);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (double)e4m3_value(a[(size_t)i * k + kk]) * std::ldexp(1.0, sa[(size_t)i * kg + kk / 32] - 127) *
                     e4m3_value(b[(size_t)j * k + kk]) * std::ldexp(1.0, sb[(size_t)j * kg + kk / 32] - 127);
            golden[(size_t)i * n + j] = (float)s;
        }
    DeviceBuffer da(a.data(), a.size()), db(b.data(), b.size()), dsa(sa.data(), sa.size()), dsb(sb.data(), sb.size()), dc((size_t)m * n * 4);
    RT(ptoamd_gemm_mx(dc.dev, PTOAMD_F32, da.dev, db.dev, PTOAMD_E4M3, PTOAMD_E4M3, (const uint8_t*)dsa.dev, (const uint8_t*)dsb.dev,
                      PTOAMD_MX_A_ND, PTOAMD_MX_B_DN, nullptr, m, n, k, k, k, n, PTOAMD_B_DN, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto out = dc.download<float>((size_t)m * n);
    printf("kernel: %s\n", ptoamd_last_kernel());
    return ResultCmp(golden, out.data(), 0.001f);
}

// quantise two f32 matrices to MXFP8, multiply the codes, and compare with the product of the de-quantised values (which
// is what the codes mean): the error against the unquantised product is the format's, not the kernel's
static bool case_quant_gemm(void* stream)
{
    const int m = 64, n = 128, k = 256, kg = k / 32;
    std::mt19937 rng(24);
    std::normal_distribution<float> d(0.0f, 1.0f);
    std::vector<float> a((size_t)m * k), b((size_t)n * k), golden((size_t)m * n);
    for (auto& v : a)
        v = d(rng);
    for (auto& v : b)
        v = d(rng);
    DeviceBuffer da(a.data(), a.size() * 4), db(b.data(), b.size() * 4), qa(a.size()), qb(b.size()), ea((size_t)m * kg), eb((size_t)n * kg),
        dc((size_t)m * n * 4);
    RT(ptoamd_tquant_mx((uint8_t*)qa.dev, (uint8_t*)ea.dev, nullptr, nullptr, da.dev, PTOAMD_F32, m, k, PTOAMD_OCP_MXFP8, 1, stream));
    RT(ptoamd_tquant_mx((uint8_t*)qb.dev, (uint8_t*)eb.dev, nullptr, nullptr, db.dev, PTOAMD_F32, n, k, PTOAMD_OCP_MXFP8, 1, stream));
    RT(ptoamd_gemm_mx(dc.dev, PTOAMD_F32, qa.dev, qb.dev, PTOAMD_E4M3, PTOAMD_E4M3, (const uint8_t*)ea.dev, (const uint8_t*)eb.dev,
                      PTOAMD_MX_A_ND, PTOAMD_MX_B_DN, nullptr, m, n, k, k, k, n, PTOAMD_B_DN, stream));
    RT(aclrtSynchronizeStream(stream));
    const auto ca = qa.download<uint8_t>(a.size()), cb = qb.download<uint8_t>(b.size());
    const auto xa = ea.download<uint8_t>((size_t)m * kg), xb = eb.download<uint8_t>((size_t)n * kg);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int kk = 0; kk < k; ++kk)
                s += (double)e4m3_value(ca[(size_t)i * k + kk]) * std::ldexp(1.0, xa[(size_t)i * kg + kk / 32] - 127) *
                     e4m3_value(cb[(size_t)j * k + kk]) * std::ldexp(1.0, xb[(size_t)j * kg + kk / 32] - 127);
            golden[(size_t)i * n + j] = (float)s;
        }
    const auto out = dc.download<float>((size_t)m * n);
    return ResultCmp(golden, out.data(), 0.001f);
}

// ---- data-driven cases ------------------------------------------------------------------------------------------------------
#include <fstream>
#include <sstream>

struct CaseLine {
    std::string suite, name, op, at, bt, ct, extra, pto;
    int m, k, n;
    float eps;
};

static int type_code(const std::string& t)
{
    static const char* names[] = {"f32", "f16", "bf16", "i32", "i8", "u8", "e4m3", "e5m2", "e2m1", "e1m2", "i16"};
    for (int i = 0; i < 11; ++i)
        if (t == names[i])
            return i;
    fprintf(stderr, "unknown type %s\n", t.c_str());
    exit(2);
}
static size_t type_bits(int t) { return (t == PTOAMD_F32 || t == PTOAMD_I32) ? 32 : ((t == PTOAMD_F16 || t == PTOAMD_BF16 || t == PTOAMD_I16) ? 16 : ((t == PTOAMD_E2M1 || t == PTOAMD_E1M2) ? 4 : 8)); }

static std::vector<uint8_t> read_bin(const std::string& dir, const CaseLine& c, const char* name, size_t expect_bytes)
{
    const std::string path = dir + "/" + c.suite + "/" + c.name + "/" + name + ".bin";
    std::ifstream f(path, std::ios::binary);
    if (!f) {
        fprintf(stderr, "cannot read %s\n", path.c_str());
        exit(2);
    }
    std::vector<uint8_t> v((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (expect_bytes != 0 && v.size() != expect_bytes) {
        fprintf(stderr, "%s holds %zu bytes, the case needs %zu\n", path.c_str(), v.size(), expect_bytes);
        exit(2);
    }
    return v;
}

static float half_value(uint16_t b)
{
    _Float16 h;
    memcpy(&h, &b, 2);
    return (float)h;
}
static float bf16_value(uint16_t b)
{
    const uint32_t w = (uint32_t)b << 16;
    float f;
    memcpy(&f, &w, 4);
    return f;
}
// rows x cols elements of type t starting at p (row pitch ld elements) as floats
static std::vector<float> as_floats(const uint8_t* p, int t, int rows, int cols, int ld)
{
    std::vector<float> v((size_t)rows * cols);
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            const size_t i = (size_t)r * ld + c;
            float x;
            switch (t) {
                case PTOAMD_F32: x = reinterpret_cast<const float*>(p)[i]; break;
                case PTOAMD_I32: x = (float)reinterpret_cast<const int32_t*>(p)[i]; break;
                case PTOAMD_F16: x = half_value(reinterpret_cast<const uint16_t*>(p)[i]); break;
                case PTOAMD_BF16: x = bf16_value(reinterpret_cast<const uint16_t*>(p)[i]); break;
                case PTOAMD_I16: x = (float)reinterpret_cast<const int16_t*>(p)[i]; break;
                case PTOAMD_U8: x = (float)p[i]; break;
                default: x = (float)reinterpret_cast<const int8_t*>(p)[i]; break;
            }
            v[(size_t)r * cols + c] = x;
        }
    return v;
}

static bool check(const CaseLine& c, const char* backend, const DeviceBuffer& out, int ct, int rows, int cols, int ld,
                  const std::vector<uint8_t>& golden)
{
    const auto raw = out.download<uint8_t>((size_t)rows * ld * type_bits(ct) / 8);
    const auto got = as_floats(raw.data(), ct, rows, cols, ld);
    const auto want = as_floats(golden.data(), ct, rows, cols, cols);
    printf("%s.%s [%s] ", c.suite.c_str(), c.name.c_str(), backend);
    return ResultCmp(want, got.data(), c.eps);
}

static bool run_data_case(const std::string& dir, const CaseLine& c, void* stream)
{
    const int at = type_code(c.at), bt = type_code(c.bt), ct = type_code(c.ct);
    const int m = c.m, k = c.k, n = c.n;
    bool ok = true;
    if (c.op == "gemm" || c.op == "gemm_bias" || c.op == "gemm_splitk" || c.op == "store" || c.op == "store_q") {
        const int repeats = c.op == "gemm_splitk" ? atoi(c.extra.c_str()) : 1;
        const auto a = read_bin(dir, c, "x1_gm", (size_t)repeats * m * k * type_bits(at) / 8);
        const auto b = read_bin(dir, c, "x2_gm", (size_t)repeats * k * n * type_bits(bt) / 8);
        const auto golden = read_bin(dir, c, "golden", (size_t)m * n * type_bits(ct) / 8);
        DeviceBuffer da(a.data(), a.size()), db(b.data(), b.size()), dc((size_t)m * n * 4), dc2((size_t)m * n * 4);
        const size_t abytes = (size_t)m * k * type_bits(at) / 8, bbytes = (size_t)k * n * type_bits(bt) / 8;
        const DeviceBuffer* result = &dc;
        if (c.op == "gemm") {
            RT(ptoamd_gemm(dc.dev, ct, da.dev, db.dev, at, nullptr, m, n, k, k, n, n, PTOAMD_B_ND, 0, stream));
        } else if (c.op == "gemm_bias") {
            const auto bias = read_bin(dir, c, "bias_gm", (size_t)n * 4);
            DeviceBuffer dbias(bias.data(), bias.size());
            RT(ptoamd_gemm_bias(dc.dev, ct, da.dev, db.dev, at, nullptr, dbias.dev, m, n, k, k, n, n, PTOAMD_B_ND, 0, stream));
            RT(aclrtSynchronizeStream(stream));
        } else if (c.op == "gemm_splitk") {  // TMATMUL for the first K slab, TMATMUL_ACC for the others
            for (int r = 0; r < repeats; ++r) {
                const DeviceBuffer& dst = (r & 1) ? dc2 : dc;
                const DeviceBuffer& src = (r & 1) ? dc : dc2;
                RT(ptoamd_gemm(dst.dev, ct, (uint8_t*)da.dev + r * abytes, (uint8_t*)db.dev + r * bbytes, at, r ? src.dev : nullptr, m, n, k, k, n,
                               n, PTOAMD_B_ND, 0, stream));
                result = &dst;
            }
        } else if (c.op == "store") {
            RT(ptoamd_gemm(dc.dev, ct, da.dev, db.dev, at, nullptr, m, n, k, k, n, n, PTOAMD_B_ND, atoi(c.extra.c_str()), stream));
        } else {
            uint64_t word = 0;
            int relu = 0;
            sscanf(c.extra.c_str(), "%llu:%d", (unsigned long long*)&word, &relu);
            DeviceBuffer dw(&word, 8);
            RT(ptoamd_gemm_requant(dc.dev, ct, da.dev, db.dev, at, nullptr, nullptr, (const uint64_t*)dw.dev, 0, m, n, k, k, n, n, PTOAMD_B_ND,
                                   relu, stream));
            RT(aclrtSynchronizeStream(stream));
        }
        RT(aclrtSynchronizeStream(stream));
        ok = check(c, ptoamd_last_kernel(), *result, ct, m, n, n, golden) && ok;
        if (c.pto.size() > 1 && c.pto[0] == 'k') {  // the same case as a kernel written in the tile ISA
            DeviceBuffer dp((size_t)m * n * 4);
            std::vector<uint8_t> bias;
            if (c.op == "gemm_bias")
                bias = read_bin(dir, c, "bias_gm", (size_t)n * 4);
            DeviceBuffer dbias(bias.empty() ? a.data() : bias.data(), bias.empty() ? 16 : bias.size());
            RT(pto_kernels_launch(atoi(c.pto.c_str() + 1), dp.dev, da.dev, db.dev, bias.empty() ? nullptr : dbias.dev, stream));
            RT(aclrtSynchronizeStream(stream));
            ok = pto_kernels_status() == 0 && check(c, "pto kernel", dp, ct, m, n, n, golden) && ok;
        }
    } else if (c.op == "mx" || c.op == "mx_bias") {
        int vm = 0, vk = 0, vn = 0;
        char fa[8] = "", fb[8] = "";
        sscanf(c.extra.c_str(), "%d:%d:%d:%7[^:]:%7s", &vm, &vk, &vn, fa, fb);
        const size_t kg = (size_t)k / 32;
        const auto a = read_bin(dir, c, "x1_gm", (size_t)m * k * type_bits(at) / 8);
        const auto b = read_bin(dir, c, "x2_gm", (size_t)n * k * type_bits(bt) / 8);
        const auto sa = read_bin(dir, c, "x1_mx_gm", (size_t)m * kg), sb = read_bin(dir, c, "x2_mx_gm", (size_t)n * kg);
        const auto golden = read_bin(dir, c, "golden", (size_t)vm * vn * 4);
        DeviceBuffer da(a.data(), a.size()), db(b.data(), b.size()), dsa(sa.data(), sa.size()), dsb(sb.data(), sb.size()), dc((size_t)m * n * 4);
        const int la = strcmp(fa, "zz") == 0 ? PTOAMD_MX_A_ZZ : PTOAMD_MX_A_ND, lb = strcmp(fb, "nn") == 0 ? PTOAMD_MX_B_NN : PTOAMD_MX_B_DN;
        if (c.op == "mx") {
            RT(ptoamd_gemm_mx(dc.dev, PTOAMD_F32, da.dev, db.dev, at, bt, (const uint8_t*)dsa.dev, (const uint8_t*)dsb.dev, la, lb, nullptr, m, n, k,
                              k, k, n, PTOAMD_B_DN, stream));
            RT(aclrtSynchronizeStream(stream));
        } else {
            const auto bias = read_bin(dir, c, "bias_gm", (size_t)n * 4);
            DeviceBuffer dbias(bias.data(), bias.size());
            RT(ptoamd_gemm_mx_bias(dc.dev, PTOAMD_F32, da.dev, db.dev, at, bt, (const uint8_t*)dsa.dev, (const uint8_t*)dsb.dev, la, lb, nullptr,
                                   (const float*)dbias.dev, m, n, k, k, k, n, PTOAMD_B_DN, stream));
            RT(aclrtSynchronizeStream(stream));
        }
        ok = check(c, ptoamd_last_kernel(), dc, PTOAMD_F32, vm, vn, n, golden);
    } else if (c.op == "storeq_tile") {  // a Vec tile through the quantising TSTORE, as a kernel written in the tile ISA
        int id = 0, sat = 0;
        sscanf(c.extra.c_str(), "%d:%d", &id, &sat);
        const size_t count = (size_t)m * n;
        const auto src = read_bin(dir, c, "input", count * type_bits(at) / 8), words = read_bin(dir, c, "quant", 0);
        const auto golden = read_bin(dir, c, "golden", count * type_bits(ct) / 8);
        DeviceBuffer ds(src.data(), src.size()), dw(words.data(), words.size()), dc(count * 4);
        RT(pto_store_quant_launch(id, dc.dev, ds.dev, dw.dev, sat, stream));
        RT(aclrtSynchronizeStream(stream));
        // (source, output and golden share one memory order, row by row or column by column: compared as a flat run)
        ok = pto_store_quant_status() == 0 && check(c, "pto kernel", dc, ct, 1, (int)count, (int)count, golden);
    } else if (c.op == "tquant_mx") {
        int alg = 0, nz = 0;
        sscanf(c.extra.c_str(), "%d:%d", &alg, &nz);
        const bool fp4 = alg >= 2;
        const size_t count = (size_t)m * n, code_bytes = fp4 ? count / 2 : count, groups = count / 32;
        const auto src = read_bin(dir, c, "input", count * type_bits(at) / 8);
        const auto golden = read_bin(dir, c, "golden", code_bytes), golden_exp = read_bin(dir, c, "golden_exp", groups);
        DeviceBuffer ds(src.data(), src.size()), dcodes(code_bytes + 16), dexp(groups + 16), dzz(groups + 16);
        RT(ptoamd_tquant_mx((uint8_t*)dcodes.dev, (uint8_t*)dexp.dev, nullptr, nullptr, ds.dev, at, m, n, alg, 1, stream));
        if (nz)  // the exponents in 16-row x 2-group boxes (the NZ store mode of TQUANT<MXFP8>)
            RT(ptoamd_mx_scale_relayout((uint8_t*)dzz.dev, PTOAMD_MX_A_ZZ, (const uint8_t*)dexp.dev, PTOAMD_MX_A_ND, m, n / 32, stream));
        RT(aclrtSynchronizeStream(stream));
        ok = check(c, "codes", dcodes, PTOAMD_U8, 1, (int)code_bytes, (int)code_bytes, golden);
        ok = check(c, "exponents", nz ? dzz : dexp, PTOAMD_U8, 1, (int)groups, (int)groups, golden_exp) && ok;
    } else if (c.op == "tquant_i8") {
        const bool asym = atoi(c.extra.c_str()) != 0;
        const size_t count = (size_t)m * n;
        const auto src = read_bin(dir, c, "input", count * 4), scale = read_bin(dir, c, "scale", (size_t)m * 4);
        const auto golden = read_bin(dir, c, "golden", count);
        std::vector<uint8_t> off;
        if (asym)
            off = read_bin(dir, c, "offset", (size_t)m * 4);
        DeviceBuffer ds(src.data(), src.size()), dsc(scale.data(), scale.size()), dof(asym ? off.data() : scale.data(), (size_t)m * 4), dc(count + 16);
        RT(ptoamd_tquant_int8(dc.dev, (const float*)ds.dev, (const float*)dsc.dev, asym ? (const float*)dof.dev : nullptr, m, n, stream));
        RT(aclrtSynchronizeStream(stream));
        ok = check(c, ptoamd_last_kernel(), dc, ct, m, n, n, golden);
    } else if (c.op == "dequant") {
        const auto src = read_bin(dir, c, "x1_gm", (size_t)m * n * type_bits(at) / 8);
        const auto scale = read_bin(dir, c, "x2_gm", (size_t)m * 4), off = read_bin(dir, c, "bias_gm", (size_t)m * 4);
        const auto golden = read_bin(dir, c, "golden", (size_t)m * n * 4);
        DeviceBuffer ds(src.data(), src.size()), dsc(scale.data(), scale.size()), dof(off.data(), off.size()), dc((size_t)m * n * 4);
        RT(ptoamd_tdequant((float*)dc.dev, ds.dev, at, (const float*)dsc.dev, (const float*)dof.dev, m, n, stream));
        RT(aclrtSynchronizeStream(stream));
        ok = check(c, ptoamd_last_kernel(), dc, PTOAMD_F32, m, n, n, golden);
    } else {
        fprintf(stderr, "unknown op %s\n", c.op.c_str());
        exit(2);
    }
    printf("%s.%s: %s\n", c.suite.c_str(), c.name.c_str(), ok ? "PASS" : "FAIL");
    return ok;
}

static int run_data_cases(int argc, char** argv)
{
    std::string dir, manifest;
    std::vector<std::string> select;
    bool list = false;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        if (a == "--data" && i + 1 < argc)
            dir = argv[++i];
        else if (a == "--manifest" && i + 1 < argc)
            manifest = argv[++i];
        else if (a == "-t" && i + 1 < argc)
            select.push_back(argv[++i]);
        else if (a == "-l")
            list = true;
        else {
            fprintf(stderr, "usage: case_runner --data <dir> --manifest <file> [-l] [-t <suite>[.<case>]]...\n");
            return 2;
        }
    }
    std::ifstream mf(manifest);
    if (!mf) {
        fprintf(stderr, "cannot read the manifest %s\n", manifest.c_str());
        return 2;
    }
    std::vector<CaseLine> cases;
    for (std::string text; std::getline(mf, text);) {
        if (text.empty() || text[0] == '#')
            continue;
        std::istringstream in(text);
        CaseLine c;
        in >> c.suite >> c.name >> c.op >> c.m >> c.k >> c.n >> c.at >> c.bt >> c.ct >> c.extra >> c.eps >> c.pto;
        if (!in) {
            fprintf(stderr, "bad manifest line: %s\n", text.c_str());
            return 2;
        }
        cases.push_back(c);
    }
    auto wanted = [&](const CaseLine& c) {
        if (select.empty())
            return true;
        for (const auto& s : select)
            if (s == c.suite || s == c.suite + "." + c.name)
                return true;
        return false;
    };
    if (list) {
        for (const auto& c : cases)
            if (wanted(c))
                printf("%s.%s\n", c.suite.c_str(), c.name.c_str());
        return 0;
    }
    aclInit(nullptr);
    RT(aclrtSetDevice(0));
    aclrtStream stream;
    RT(aclrtCreateStream(&stream));
    int ran = 0, failed = 0;
    for (const auto& c : cases)
        if (wanted(c)) {
            ++ran;
            failed += run_data_case(dir, c, stream) ? 0 : 1;
        }
    aclrtDestroyStream(stream);
    aclrtResetDevice(0);
    aclFinalize();
    printf("%d cases run, %d failed\n", ran, failed);
    if (ran == 0) {
        fprintf(stderr, "no case matches the selection\n");
        return 2;
    }
    return failed ? 1 : 0;
}

int main(int argc, char** argv)
{
    if (argc > 1 && (strcmp(argv[1], "--data") == 0 || strcmp(argv[1], "--manifest") == 0 || strcmp(argv[1], "-l") == 0 ||
                     strcmp(argv[1], "-t") == 0))
        return run_data_cases(argc, argv);
    if (argc != 2) {
        fprintf(stderr, "usage: case_runner tmatmul|tmatmul_i8|tmatmul_mx|gemm|gemm_mx|quant_gemm\n");
        return 2;
    }
    const std::string name = argv[1];
    aclInit(nullptr);
    RT(aclrtSetDevice(0));
    aclrtStream stream;
    RT(aclrtCreateStream(&stream));
    bool ok;
    if (name == "tmatmul")
        ok = case_tmatmul(stream);
    else if (name == "tmatmul_i8")
        ok = case_tmatmul_i8(stream);
    else if (name == "tmatmul_mx")
        ok = case_tmatmul_mx(stream);
    else if (name == "gemm")
        ok = case_gemm(stream);
    else if (name == "gemm_mx")
        ok = case_gemm_mx(stream);
    else if (name == "quant_gemm")
        ok = case_quant_gemm(stream);
    else {
        fprintf(stderr, "unknown case %s\n", name.c_str());
        return 2;
    }
    aclrtDestroyStream(stream);
    aclrtResetDevice(0);
    aclFinalize();
    printf("%s: %s\n", name.c_str(), ok ? "PASS" : "FAIL");
    return ok ? 0 : 1;
}
