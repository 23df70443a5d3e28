// A test main without a test framework, in the shape of the reference's (tests/cpu/st/testcase/tmatmul/main.cpp:40-95,
// tests/cpu/st/testcase/tmatmul_mx/main.cpp:58-148): aclrt* runtime calls, host buffers filled from the reference
// generators' distributions (tmatmul/gen_data.py, tmatmul_mx/gen_data.py), one Launch call, a host-side golden and a
// comparison with the semantics of the reference's ResultCmp (tests/common/test_common.h:231-309).
//
//   case_runner <case>      exit status 0 = match, 1 = mismatch, 2 = usage / runtime error
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

int main(int argc, char** argv)
{
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
