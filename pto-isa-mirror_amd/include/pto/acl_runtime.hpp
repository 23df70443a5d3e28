// Host runtime names of a PTO test / demo main() (aclInit, aclrtSetDevice, aclrtMalloc, aclrtMemcpy, ...) on top of the
// gfx950 library's C ABI (ptoamd.h).  Reference: include/pto/common/cpu_stub.hpp:64-120,524-555 (the CPU simulator's
// definitions of the same names) and tests/cpu/st/testcase/tmatmul/main.cpp:46-84 (how a test main uses them).
// All functions return 0 on success, like the reference's.
#pragma once
#include <ptoamd.h>

#include <stddef.h>

using aclrtStream = void*;

enum {
    ACL_MEM_MALLOC_HUGE_FIRST = 0,
    ACL_MEMCPY_HOST_TO_DEVICE = 0,
    ACL_MEMCPY_DEVICE_TO_HOST = 1,
    ACL_MEMCPY_DEVICE_TO_DEVICE = 2,
};

inline int aclInit(const char*) { return 0; }
inline int aclrtSetDevice(int device) { return ptoamd_init(device); }
inline int aclrtCreateStream(aclrtStream* stream) { return ptoamd_stream_create(stream); }
inline int aclrtDestroyStream(aclrtStream stream) { return ptoamd_stream_destroy(stream); }
inline int aclrtSynchronizeStream(aclrtStream stream) { return ptoamd_stream_synchronize(stream); }
inline int aclrtMallocHost(void** p, size_t bytes) { return ptoamd_malloc_host(p, bytes); }
inline int aclrtMalloc(void** p, size_t bytes, int) { return ptoamd_malloc(p, bytes); }
inline int aclrtFree(void* p) { return ptoamd_free(p); }
inline int aclrtFreeHost(void* p) { return ptoamd_free_host(p); }
inline int aclrtMemcpy(void* dst, size_t dst_bytes, const void* src, size_t count, int kind)
{
    static const int map[3] = {PTOAMD_MEMCPY_H2D, PTOAMD_MEMCPY_D2H, PTOAMD_MEMCPY_D2D};
    if (kind < 0 || kind > 2)
        return PTOAMD_E_INVALID;
    return ptoamd_memcpy(dst, dst_bytes, src, count, map[kind]);
}
inline int aclrtMemset(void* dst, size_t dst_bytes, int value, size_t count) { return ptoamd_memset(dst, dst_bytes, value, count); }
inline int aclrtResetDevice(int) { return 0; }
inline int aclFinalize() { return ptoamd_finalize(); }
