// Host runtime of the gfx950 backend: the counterpart of the fake aclrt* runtime the reference's tests and demos use
// (include/pto/common/cpu_stub.hpp:73-120, 524-555), on the HIP runtime.
#include <dlfcn.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <mutex>
#include <set>
#include <utility>

#include "common_host.hpp"

namespace ptoamd {
static thread_local char g_error[512] = "";
static thread_local char g_kernel[64] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}
static thread_local unsigned long g_launches = 0;
void set_last_kernel(const char* name)
{
    strncpy(g_kernel, name, sizeof g_kernel - 1);
    g_kernel[sizeof g_kernel - 1] = 0;
    ++g_launches;
}

// ---- environment switches ---------------------------------------------------------------------------------------------
namespace {
Options g_options;
std::once_flag g_options_once;
bool env_is_1(const char* name)
{
    const char* v = getenv(name);
    return v != nullptr && v[0] == '1';
}
void read_options()
{
    Options o;
    const char* t = getenv("PTOAMD_TILE");
    if (t != nullptr && t[0] >= '0' && t[0] <= '7')
        o.tile = t[0] - '0';
    o.no_tail_split = getenv("PTOAMD_NO_TAIL_SPLIT") != nullptr;
    o.mx_16x16 = getenv("PTOAMD_MX_16X16") != nullptr;
    const char* tt = getenv("PTOAMD_TAIL_TILE");
    if (tt != nullptr && tt[0] >= '5' && tt[0] <= '7')
        o.tail_tile = tt[0] - '0';
    o.force_generic = env_is_1("PTOAMD_FORCE_GENERIC");
    o.b_nd_in_loader = getenv("PTOAMD_B_ND_IN_LOADER") != nullptr;
    o.gemv_sw_cvt = env_is_1("PTOAMD_GEMV_SW_CVT");
    o.gemv_no_splitk = env_is_1("PTOAMD_GEMV_NO_SPLITK");
    o.gemv_no_wide = env_is_1("PTOAMD_GEMV_NO_WIDE");
    g_options = o;
}
}  // namespace
const Options& options()
{
    std::call_once(g_options_once, read_options);
    return g_options;
}
int device_compute_units()
{
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 256;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

// ---- launch trace -----------------------------------------------------------------------------------------------------
namespace {
struct TraceSink {
    std::mutex mu;
    FILE* file = nullptr;
    unsigned long sequence = 0;
    bool enabled = false;
    TraceSink()
    {
        const char* dir = getenv("PTOAMD_TRACE_DIR");
        if (dir == nullptr || *dir == 0)
            return;
        char path[1024];
        snprintf(path, sizeof path, "%s/ptoamd_trace_%ld.jsonl", dir, (long)getpid());
        file = fopen(path, "a");
        enabled = file != nullptr;
    }
    ~TraceSink()
    {
        if (file)
            fclose(file);
    }
};
TraceSink& trace_sink()
{
    static TraceSink sink;
    return sink;
}

// Marker ranges for profilers (PTOAMD_ROCTX=1): every C-ABI launch is bracketed by a roctx range named after the PTO
// instruction chain it stands for, so `rocprofv3 --marker-trace --kernel-trace` shows PTO opcodes next to the kernels.
// The marker library is looked up at run time (rocprofiler-sdk's, else roctracer's); without it the switch does nothing.
struct Roctx {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    Roctx()
    {
        const char* on = getenv("PTOAMD_ROCTX");
        if (on == nullptr || on[0] != '1')
            return;
        for (const char* name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
            void* h = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
            if (h == nullptr)
                continue;
            push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
            pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
            if (push != nullptr && pop != nullptr)
                return;
            push = nullptr;
            pop = nullptr;
        }
    }
};
Roctx& roctx()
{
    static Roctx r;
    return r;
}
const char* dtype_name(int t)
{
    static const char* names[] = {"f32", "f16", "bf16", "i32", "i8", "u8", "e4m3", "e5m2", "e2m1x2", "e1m2x2", "i16"};
    return t >= 0 && t < 11 ? names[t] : (t == 100 ? "e8m0" : (t == 101 ? "u64" : "?"));
}
}  // namespace

TraceScope::TraceScope(const char* opcode, const char* pipeline, long m, long n, long k)
    : on_(trace_sink().enabled), opcode_(opcode), pipeline_(pipeline), m_(m), n_(n), k_(k), launches_before_(g_launches)
{
    if (roctx().push != nullptr) {
        char label[96];
        snprintf(label, sizeof label, "PTO %s %ldx%ldx%ld", opcode, m, n, k);
        roctx().push(label);
    }
}
TraceScope& TraceScope::in(const void* address, long rows, long cols, const char* layout, int dtype)
{
    if (on_ && address != nullptr && nin_ < 6)
        in_[nin_++] = Tile{address, rows, cols, layout, dtype};
    return *this;
}
TraceScope& TraceScope::out(const void* address, long rows, long cols, const char* layout, int dtype)
{
    if (on_ && address != nullptr && nout_ < 4)
        out_[nout_++] = Tile{address, rows, cols, layout, dtype};
    return *this;
}
TraceScope::~TraceScope()
{
    if (roctx().pop != nullptr)
        roctx().pop();
    if (!on_ || g_launches == launches_before_)
        return;  // tracing off, or the call was rejected before anything ran
    TraceSink& sink = trace_sink();
    std::lock_guard<std::mutex> lock(sink.mu);
    fprintf(sink.file, "{\"sequence_id\": %lu, \"opcode\": \"%s\", \"pipeline\": \"%s\", \"kernel\": \"%s\", \"m\": %ld, \"n\": %ld, \"k\": %ld",
            sink.sequence++, opcode_, pipeline_, g_kernel, m_, n_, k_);
    for (int side = 0; side < 2; ++side) {
        const Tile* t = side == 0 ? in_ : out_;
        const int cnt = side == 0 ? nin_ : nout_;
        fprintf(sink.file, ", \"%s\": [", side == 0 ? "input_tiles" : "output_tiles");
        for (int i = 0; i < cnt; ++i)
            fprintf(sink.file, "%s{\"address\": %llu, \"shape\": [%ld, %ld], \"layout\": \"%s\", \"dtype\": \"%s\"}", i ? ", " : "",
                    (unsigned long long)(uintptr_t)t[i].address, t[i].rows, t[i].cols, t[i].layout, dtype_name(t[i].dtype));
        fprintf(sink.file, "]");
    }
    fprintf(sink.file, "}\n");
    fflush(sink.file);
}

// hipFuncAttributeMaxDynamicSharedMemorySize is a property of (kernel, device): it is set once per pair, under a lock,
// so that launches from several host threads or on several devices of one process all see it.
hipError_t ensure_dynamic_lds(const void* kernel, int bytes)
{
    static std::mutex mu;
    static std::set<std::pair<int, const void*>> done;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    std::lock_guard<std::mutex> lock(mu);
    const auto key = std::make_pair(dev, kernel);
    if (done.count(key))
        return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess)
        done.insert(key);
    return e;
}
}  // namespace ptoamd

using namespace ptoamd;

extern "C" {

const char* ptoamd_last_error(void) { return g_error; }
const char* ptoamd_last_kernel(void) { return g_kernel; }

int ptoamd_init(int device)
{
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        set_error("no HIP device visible");
        return PTOAMD_E_NODEVICE;
    }
    PTOAMD_REQUIRE(device >= 0 && device < count, PTOAMD_E_INVALID, "device %d out of range (0..%d)", device, count - 1);
    PTOAMD_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    PTOAMD_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
        return PTOAMD_E_NODEVICE;
    }
    (void)options();
    (void)device_compute_units();
    int rc = prepare_gemm_kernels();
    if (rc == PTOAMD_OK)
        rc = prepare_gemv_kernels();
    return rc;
}

int ptoamd_reload_options(void)
{
    (void)options();   // the first read has happened
    read_options();    // not synchronised with launches running on other host threads: call it between launches
    return PTOAMD_OK;
}

int ptoamd_finalize(void)
{
    PTOAMD_HIP_CHECK(hipDeviceSynchronize());
    return PTOAMD_OK;
}

int ptoamd_device_info(int* compute_units, int* clock_khz, size_t* hbm_bytes, char* arch, size_t arch_len)
{
    int dev = 0;
    PTOAMD_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    PTOAMD_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (compute_units)
        *compute_units = prop.multiProcessorCount;
    if (clock_khz)
        *clock_khz = prop.clockRate;
    if (hbm_bytes)
        *hbm_bytes = prop.totalGlobalMem;
    if (arch && arch_len) {
        strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return PTOAMD_OK;
}

int ptoamd_malloc(void** dev_ptr, size_t bytes)
{
    PTOAMD_REQUIRE(dev_ptr != nullptr && bytes > 0, PTOAMD_E_INVALID, "ptoamd_malloc: null result pointer or zero size");
    PTOAMD_HIP_CHECK(hipMalloc(dev_ptr, bytes));
    return PTOAMD_OK;
}
int ptoamd_free(void* dev_ptr)
{
    PTOAMD_HIP_CHECK(hipFree(dev_ptr));
    return PTOAMD_OK;
}
int ptoamd_malloc_host(void** host_ptr, size_t bytes)
{
    PTOAMD_REQUIRE(host_ptr != nullptr && bytes > 0, PTOAMD_E_INVALID, "ptoamd_malloc_host: null result pointer or zero size");
    PTOAMD_HIP_CHECK(hipHostMalloc(host_ptr, bytes, hipHostMallocDefault));
    return PTOAMD_OK;
}
int ptoamd_free_host(void* host_ptr)
{
    PTOAMD_HIP_CHECK(hipHostFree(host_ptr));
    return PTOAMD_OK;
}

static int to_kind(int kind, hipMemcpyKind* out)
{
    switch (kind) {
        case PTOAMD_MEMCPY_H2H: *out = hipMemcpyHostToHost; return 0;
        case PTOAMD_MEMCPY_H2D: *out = hipMemcpyHostToDevice; return 0;
        case PTOAMD_MEMCPY_D2H: *out = hipMemcpyDeviceToHost; return 0;
        case PTOAMD_MEMCPY_D2D: *out = hipMemcpyDeviceToDevice; return 0;
        default: return -1;
    }
}

int ptoamd_memcpy(void* dst, size_t dst_bytes, const void* src, size_t count, int kind)
{
    hipMemcpyKind k;
    PTOAMD_REQUIRE(to_kind(kind, &k) == 0, PTOAMD_E_INVALID, "ptoamd_memcpy: unknown kind %d", kind);
    PTOAMD_REQUIRE(count <= dst_bytes, PTOAMD_E_INVALID, "ptoamd_memcpy: count %zu exceeds destination size %zu", count,
                   dst_bytes);
    if (count == 0)
        return PTOAMD_OK;
    PTOAMD_REQUIRE(dst != nullptr && src != nullptr, PTOAMD_E_INVALID, "ptoamd_memcpy: null pointer");
    PTOAMD_HIP_CHECK(hipMemcpy(dst, src, count, k));
    return PTOAMD_OK;
}
int ptoamd_memcpy_async(void* dst, size_t dst_bytes, const void* src, size_t count, int kind, void* stream)
{
    hipMemcpyKind k;
    PTOAMD_REQUIRE(to_kind(kind, &k) == 0, PTOAMD_E_INVALID, "ptoamd_memcpy_async: unknown kind %d", kind);
    PTOAMD_REQUIRE(count <= dst_bytes, PTOAMD_E_INVALID, "ptoamd_memcpy_async: count %zu exceeds destination size %zu",
                   count, dst_bytes);
    if (count == 0)
        return PTOAMD_OK;
    PTOAMD_REQUIRE(dst != nullptr && src != nullptr, PTOAMD_E_INVALID, "ptoamd_memcpy_async: null pointer");
    PTOAMD_HIP_CHECK(hipMemcpyAsync(dst, src, count, k, as_stream(stream)));
    return PTOAMD_OK;
}
int ptoamd_memset(void* dev_ptr, size_t dst_bytes, int value, size_t count)
{
    PTOAMD_REQUIRE(count <= dst_bytes, PTOAMD_E_INVALID, "ptoamd_memset: count %zu exceeds destination size %zu", count,
                   dst_bytes);
    if (count == 0)
        return PTOAMD_OK;
    PTOAMD_REQUIRE(dev_ptr != nullptr, PTOAMD_E_INVALID, "ptoamd_memset: null pointer");
    PTOAMD_HIP_CHECK(hipMemset(dev_ptr, value, count));
    return PTOAMD_OK;
}

int ptoamd_stream_create(void** stream)
{
    PTOAMD_REQUIRE(stream != nullptr, PTOAMD_E_INVALID, "ptoamd_stream_create: null result pointer");
    hipStream_t s;
    PTOAMD_HIP_CHECK(hipStreamCreate(&s));
    *stream = s;
    return PTOAMD_OK;
}
int ptoamd_stream_destroy(void* stream)
{
    PTOAMD_HIP_CHECK(hipStreamDestroy(as_stream(stream)));
    return PTOAMD_OK;
}
int ptoamd_stream_synchronize(void* stream)
{
    PTOAMD_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
    return PTOAMD_OK;
}

int ptoamd_event_create(void** event)
{
    PTOAMD_REQUIRE(event != nullptr, PTOAMD_E_INVALID, "ptoamd_event_create: null result pointer");
    hipEvent_t e;
    PTOAMD_HIP_CHECK(hipEventCreate(&e));
    *event = e;
    return PTOAMD_OK;
}
int ptoamd_event_destroy(void* event)
{
    PTOAMD_HIP_CHECK(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return PTOAMD_OK;
}
int ptoamd_event_record(void* event, void* stream)
{
    PTOAMD_HIP_CHECK(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
    return PTOAMD_OK;
}
int ptoamd_event_synchronize(void* event)
{
    PTOAMD_HIP_CHECK(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return PTOAMD_OK;
}
int ptoamd_event_elapsed_ms(float* ms, void* start, void* stop)
{
    PTOAMD_REQUIRE(ms != nullptr, PTOAMD_E_INVALID, "ptoamd_event_elapsed_ms: null result pointer");
    PTOAMD_HIP_CHECK(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return PTOAMD_OK;
}

}  // extern "C"
