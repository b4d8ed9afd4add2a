// Device selection, error text and the thin memory helpers of the C ABI.
#include <atomic>
#include <mutex>

#include "common.h"

namespace vsag_amd {

char*
last_error_buffer() {
    static thread_local char buf[1024] = {0};
    return buf;
}

static std::mutex g_init_mutex;
static std::atomic<int> g_device{-1};
static int g_cu_count = 0;
static char g_name[256] = {0};
static uint64_t g_hbm = 0;

int static_scratch_setup(int device);  // scan.hip: address of the library's own scratch array on `device`

__global__ void
probe_kernel(int* out) {
    *out = 950;
}

static int
init_device(int device) {
    int count = 0;
    hipError_t err = hipGetDeviceCount(&count);
    if (err != hipSuccess || count == 0) {
        return fail(VSAG_AMD_INTERNAL_ERROR,
                    "no HIP device available (%s); this library has no CPU fallback",
                    err == hipSuccess ? "device count is 0" : hipGetErrorString(err));
    }
    VA_CHECK_ARG(device >= 0 && device < count, "device %d out of range [0, %d)", device, count);
    VA_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    VA_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        return fail(VSAG_AMD_INTERNAL_ERROR, "device %d is %s; the kernels are built for gfx950 only", device,
                    prop.gcnArchName);
    }
    // Launch one trivial kernel so that a missing / mismatched code object is reported here, loudly.
    int* flag = nullptr;
    VA_HIP(hipMalloc(&flag, sizeof(int)));
    hipLaunchKernelGGL(probe_kernel, dim3(1), dim3(1), 0, nullptr, flag);
    hipError_t launch = hipGetLastError();
    int host_flag = 0;
    hipError_t copy = hipMemcpy(&host_flag, flag, sizeof(int), hipMemcpyDeviceToHost);
    (void)hipFree(flag);
    if (launch != hipSuccess || copy != hipSuccess || host_flag != 950) {
        return fail(VSAG_AMD_INTERNAL_ERROR, "gfx950 code object did not load or run: %s",
                    hipGetErrorString(launch != hipSuccess ? launch : copy));
    }
    VA_TRY(static_scratch_setup(device));
    g_cu_count = prop.multiProcessorCount;
    g_hbm = prop.totalGlobalMem;
    snprintf(g_name, sizeof(g_name), "%s (%s)", prop.name, prop.gcnArchName);
    g_device.store(device);
    return 0;
}

int
ensure_init() {
    if (g_device.load() >= 0) {
        return 0;
    }
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_device.load() >= 0) {
        return 0;
    }
    int current = 0;
    if (hipGetDevice(&current) != hipSuccess) {
        current = 0;
    }
    return init_device(current);
}

int
device_cu_count() {
    return g_cu_count > 0 ? g_cu_count : 256;
}

// ---- optional timing of the dominant kernel of a call (HIP events on the caller's stream) ----------
static std::atomic<int> g_timing{0};
struct KernelTimer {
    hipEvent_t start = nullptr, stop = nullptr;
    bool recorded = false;
};
static thread_local KernelTimer tl_timer;
static thread_local bool tl_timing_off = false;

// Calls that must not create anything (events included) switch the measurement hook off for their duration.
bool
timing_suppress(bool off) {
    const bool was = tl_timing_off;
    tl_timing_off = off;
    return was;
}

void
timing_begin(hipStream_t st) {
    if (g_timing.load() == 0 || tl_timing_off) {
        return;
    }
    if (tl_timer.start == nullptr) {
        if (hipEventCreate(&tl_timer.start) != hipSuccess || hipEventCreate(&tl_timer.stop) != hipSuccess) {
            return;
        }
    }
    tl_timer.recorded = hipEventRecord(tl_timer.start, st) == hipSuccess;
}

void
timing_end(hipStream_t st) {
    if (g_timing.load() == 0 || tl_timing_off || !tl_timer.recorded) {
        return;
    }
    tl_timer.recorded = hipEventRecord(tl_timer.stop, st) == hipSuccess;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" int
vsag_amd_set_kernel_timing(int enable) {
    g_timing.store(enable ? 1 : 0);
    return 0;
}

extern "C" int
vsag_amd_last_kernel_ms(float* ms) {
    VA_CHECK_ARG(ms != nullptr, "ms is null");
    VA_CHECK_ARG(tl_timer.recorded, "no timed kernel on this thread: call vsag_amd_set_kernel_timing(1) first");
    VA_HIP(hipEventSynchronize(tl_timer.stop));
    VA_HIP(hipEventElapsedTime(ms, tl_timer.start, tl_timer.stop));
    return 0;
}

extern "C" int
vsag_amd_init(int device) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    return init_device(device);
}

extern "C" const char*
vsag_amd_last_error(void) {
    return last_error_buffer();
}

extern "C" int
vsag_amd_device_info(char* name, size_t name_bytes, int* compute_units, uint64_t* hbm_bytes) {
    VA_TRY(ensure_init());
    if (name != nullptr && name_bytes > 0) {
        snprintf(name, name_bytes, "%s", g_name);
    }
    if (compute_units != nullptr) {
        *compute_units = g_cu_count;
    }
    if (hbm_bytes != nullptr) {
        *hbm_bytes = g_hbm;
    }
    return 0;
}

extern "C" int
vsag_amd_malloc(void** ptr_dev, size_t bytes) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(ptr_dev != nullptr, "ptr_dev is null");
    *ptr_dev = nullptr;
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMalloc(ptr_dev, bytes));
    return 0;
}

extern "C" int
vsag_amd_free(void* ptr_dev) {
    if (ptr_dev == nullptr) {
        return 0;
    }
    VA_HIP(hipFree(ptr_dev));
    return 0;
}

extern "C" int
vsag_amd_memory_info(uint64_t* free_bytes, uint64_t* total_bytes, uint64_t* async_pool_high_bytes, int reset_high) {
    VA_TRY(ensure_init());
    size_t f = 0, t = 0;
    VA_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes != nullptr) {
        *free_bytes = f;
    }
    if (total_bytes != nullptr) {
        *total_bytes = t;
    }
    int device = 0;
    VA_HIP(hipGetDevice(&device));
    hipMemPool_t pool = nullptr;
    VA_HIP(hipDeviceGetDefaultMemPool(&pool, device));
    if (async_pool_high_bytes != nullptr) {
        uint64_t high = 0;
        VA_HIP(hipMemPoolGetAttribute(pool, hipMemPoolAttrUsedMemHigh, &high));
        *async_pool_high_bytes = high;
    }
    if (reset_high) {
        uint64_t zero = 0;
        VA_HIP(hipMemPoolSetAttribute(pool, hipMemPoolAttrUsedMemHigh, &zero));
    }
    return 0;
}

extern "C" int
vsag_amd_memcpy_h2d(void* dst_dev, const void* src, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemcpyAsync(dst_dev, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
    VA_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" int
vsag_amd_memcpy_d2h(void* dst, const void* src_dev, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemcpyAsync(dst, src_dev, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    VA_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return 0;
}

// Pinned host memory (allocated, never registered) and copies that do not wait: what a serving loop stages its
// queries and results through, with one vsag_amd_stream_synchronize per search.
extern "C" int
vsag_amd_host_malloc(void** ptr, size_t bytes) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(ptr != nullptr, "ptr is null");
    *ptr = nullptr;
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return 0;
}

extern "C" int
vsag_amd_host_free(void* ptr) {
    if (ptr == nullptr) {
        return 0;
    }
    VA_HIP(hipHostFree(ptr));
    return 0;
}

extern "C" int
vsag_amd_memcpy_h2d_async(void* dst_dev, const void* src, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemcpyAsync(dst_dev, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" int
vsag_amd_memcpy_d2h_async(void* dst, const void* src_dev, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemcpyAsync(dst, src_dev, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" int
vsag_amd_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" int
vsag_amd_memset(void* dst_dev, int value, size_t bytes, void* stream) {
    VA_TRY(ensure_init());
    if (bytes == 0) {
        return 0;
    }
    VA_HIP(hipMemsetAsync(dst_dev, value, bytes, static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" int
vsag_amd_stream_create(void** stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(stream != nullptr, "stream is null");
    hipStream_t st = nullptr;
    // Default priority; independent of the null stream, so that searches on different streams overlap.
    VA_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *stream = st;
    return 0;
}

extern "C" int
vsag_amd_stream_destroy(void* stream) {
    if (stream != nullptr) {
        VA_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    }
    return 0;
}

extern "C" int
vsag_amd_stream_synchronize(void* stream) {
    VA_TRY(ensure_init());
    VA_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return 0;
}
