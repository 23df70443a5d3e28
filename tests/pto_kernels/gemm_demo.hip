// Host program in the shape of the reference's test mains (tests/cpu/st/testcase/tmatmul/main.cpp:40-95) and of its
// CPU-simulator GEMM demo (demos/cpu/gemm_demo/gemm_demo.cpp:83-121): aclrt* runtime calls, one Launch function, a
// host-side fp32 check.  Workload: fp16 A[512 x 512] . B[512 x 512] -> fp32 C, uniform [-1, 1] from a fixed seed,
// 128 x 128 output tiles, K walked by 64 through TLOAD / TMOV / TMATMUL_ACC / TSTORE on the gfx950 header layer.
// Prints `max_abs_diff=<x> max_rel=<y>` and exits 0 when max_rel <= 1e-2.
#include <pto/pto-inst.hpp>
#include <pto/acl_runtime.hpp>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

using namespace pto;

constexpr int M = 512, K = 512, N = 512, BM = 128, BN = 128, BK = 64;

__global__ AICORE void GemmDemoKernel(__gm__ float* out, __gm__ half* a, __gm__ half* b)
{
    constexpr int tilesN = N / BN;
    const int tile = (int)get_block_idx();
    const int tm = tile / tilesN, tn = tile % tilesN;
    using GlobalA = GlobalTensor<half, Shape<1, 1, 1, BM, BK>, Stride<M * K, M * K, M * K, K, 1>>;
    using GlobalB = GlobalTensor<half, Shape<1, 1, 1, BK, BN>, Stride<K * N, K * N, K * N, N, 1>>;
    using GlobalC = GlobalTensor<float, Shape<1, 1, 1, BM, BN>, Stride<M * N, M * N, M * N, N, 1>>;
    Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor, 512> aMat;
    Tile<TileType::Mat, half, BK, BN, BLayout::ColMajor, BK, BN, SLayout::RowMajor, 512> bMat;
    TileLeft<half, BM, BK> aTile;
    TileRight<half, BK, BN> bTile;
    TileAcc<float, BM, BN> cTile;
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, 0x8000);
    TASSIGN(aTile, 0x0);
    TASSIGN(bTile, 0x0);
    TASSIGN(cTile, 0x0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        GlobalA aGlobal(a + (size_t)tm * BM * K + k0);
        GlobalB bGlobal(b + (size_t)k0 * N + tn * BN);
        TLOAD(aMat, aGlobal);
        TLOAD(bMat, bGlobal);
        TMOV(aTile, aMat);
        TMOV(bTile, bMat);
        if (k0 == 0)
            TMATMUL(cTile, aTile, bTile);
        else
            TMATMUL_ACC(cTile, cTile, aTile, bTile);
    }
    GlobalC cGlobal(out + (size_t)tm * BM * N + tn * BN);
    TSTORE(cGlobal, cTile);
}

void LaunchGemmDemo(uint8_t* out, uint8_t* src0, uint8_t* src1, void* stream)
{
    const int rc = pto::amd::launch<&GemmDemoKernel>((M / BM) * (N / BN), stream, reinterpret_cast<float*>(out),
                                                     reinterpret_cast<half*>(src0), reinterpret_cast<half*>(src1));
    if (rc != 0) {
        fprintf(stderr, "launch failed: %d\n", rc);
        abort();
    }
}

int main()
{
    const size_t aBytes = (size_t)M * K * sizeof(half), bBytes = (size_t)K * N * sizeof(half), cBytes = (size_t)M * N * sizeof(float);
    aclInit(nullptr);
    if (aclrtSetDevice(0) != 0) {
        fprintf(stderr, "%s\n", ptoamd_last_error());
        return 2;
    }
    aclrtStream stream;
    aclrtCreateStream(&stream);
    uint8_t *dstHost, *src0Host, *src1Host, *dstDevice, *src0Device, *src1Device;
    aclrtMallocHost((void**)&dstHost, cBytes);
    aclrtMallocHost((void**)&src0Host, aBytes);
    aclrtMallocHost((void**)&src1Host, bBytes);
    aclrtMalloc((void**)&dstDevice, cBytes, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void**)&src0Device, aBytes, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void**)&src1Device, bBytes, ACL_MEM_MALLOC_HUGE_FIRST);

    std::mt19937 rng(1234);
    std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
    half* a = reinterpret_cast<half*>(src0Host);
    half* b = reinterpret_cast<half*>(src1Host);
    for (size_t i = 0; i < (size_t)M * K; ++i)
        a[i] = (half)dist(rng);
    for (size_t i = 0; i < (size_t)K * N; ++i)
        b[i] = (half)dist(rng);

    aclrtMemset(dstDevice, cBytes, 0, cBytes);
    aclrtMemcpy(src0Device, aBytes, src0Host, aBytes, ACL_MEMCPY_HOST_TO_DEVICE);
    aclrtMemcpy(src1Device, bBytes, src1Host, bBytes, ACL_MEMCPY_HOST_TO_DEVICE);
    LaunchGemmDemo(dstDevice, src0Device, src1Device, stream);
    aclrtSynchronizeStream(stream);
    aclrtMemcpy(dstHost, cBytes, dstDevice, cBytes, ACL_MEMCPY_DEVICE_TO_HOST);

    // host check: sequential fp32 fma over k, the simulator's TMATMUL arithmetic
    const float* c = reinterpret_cast<const float*>(dstHost);
    double max_abs = 0, max_ref = 0;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int k = 0; k < K; ++k)
                acc = std::fma((float)a[(size_t)i * K + k], (float)b[(size_t)k * N + j], acc);
            max_abs = std::fmax(max_abs, std::fabs((double)acc - c[(size_t)i * N + j]));
            max_ref = std::fmax(max_ref, std::fabs((double)acc));
        }
    const int status = pto::amd::device_status();
    printf("max_abs_diff=%.3e max_rel=%.3e status=%d\n", max_abs, max_abs / max_ref, status);

    aclrtFree(dstDevice);
    aclrtFree(src0Device);
    aclrtFree(src1Device);
    aclrtFreeHost(dstHost);
    aclrtFreeHost(src0Host);
    aclrtFreeHost(src1Host);
    aclrtDestroyStream(stream);
    aclrtResetDevice(0);
    aclFinalize();
    return (status == 0 && max_abs / max_ref <= 1e-2) ? 0 : 1;
}
