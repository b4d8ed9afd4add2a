// Shared host/device helpers of the gfx950 search core: error plumbing, key encoding, tile geometry.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/vsag_amd.h"

namespace vsag_amd {

constexpr int kWave = 64;          // gfx950 wavefront width; one code tile holds 64 codes
constexpr int kGranule = 16;       // bytes per lane per tile row (one dwordx4)
// Scan-kernel variant of VSAG_AMD_KIND_RABITQ for stores whose queries stay fp32 (rabitq_bits_per_dim_query = 32);
// only the kernel templates and their dispatch know it.
constexpr int kKindRabitqF32 = 100;  // a tag of the kernels only, beyond the public kinds
// pqfs: the float table of a query (16 entries per subspace) must fit 64 KB of LDS while it is quantised
constexpr uint32_t kMaxPqDim = 1024;
constexpr int kMaxGroup = 8;       // most granule rows the scans fetch together
// Readable bytes past the last tile of every tile buffer: the last group of a tile is fetched whole.
constexpr size_t kTileSlackBytes = static_cast<size_t>(kMaxGroup - 1) * kWave * kGranule;

// Granule rows fetched together by a wave that serves T queries: one query leaves registers for a deeper
// prefetch, which a wave needs when few waves share the memory latency.
template <int T>
struct GroupOf {
    static constexpr int value = T == 1 ? 8 : 4;
};
constexpr uint32_t kMaxTopK = 1024;
constexpr uint64_t kInfKey = 0xFFFFFFFFFFFFFFFFull;

// ---- error plumbing -----------------------------------------------------------------------------
char* last_error_buffer();  // thread-local, 1024 bytes

inline int
fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buffer(), 1024, fmt, ap);
    va_end(ap);
    return code;
}

#define VA_HIP(expr)                                                                                     \
    do {                                                                                                 \
        hipError_t err__ = (expr);                                                                       \
        if (err__ != hipSuccess) {                                                                       \
            return ::vsag_amd::fail(err__ == hipErrorOutOfMemory ? VSAG_AMD_NO_ENOUGH_MEMORY            \
                                                                 : VSAG_AMD_INTERNAL_ERROR,             \
                                    "%s failed: %s (%s:%d)", #expr, hipGetErrorString(err__), __FILE__, \
                                    __LINE__);                                                           \
        }                                                                                                \
    } while (0)

#define VA_CHECK_ARG(cond, ...)                                              \
    do {                                                                     \
        if (!(cond)) {                                                       \
            return ::vsag_amd::fail(VSAG_AMD_INVALID_ARGUMENT, __VA_ARGS__); \
        }                                                                    \
    } while (0)

#define VA_TRY(expr)          \
    do {                      \
        int rc__ = (expr);    \
        if (rc__ != 0) {      \
            return rc__;      \
        }                     \
    } while (0)

int ensure_init();  // VSAG_AMD_INTERNAL_ERROR when no gfx950 device is usable
int device_cu_count();

inline uint64_t
round_up(uint64_t v, uint64_t a) {
    return (v + a - 1) / a * a;
}
inline uint64_t
div_up(uint64_t v, uint64_t a) {
    return (v + a - 1) / a;
}

// The RaBitQ rotation y = R x is done for this many rows at a time, so that its temporary stays bounded.
constexpr uint64_t kRotateSlabRows = 1ull << 18;

// Carves 256-byte aligned pieces out of a caller-supplied workspace.
struct Carver {
    uint8_t* base;
    size_t size;
    size_t used = 0;
    Carver(void* p, size_t n) : base(static_cast<uint8_t*>(p)), size(n) {
    }
    template <typename T>
    T*
    take(size_t count) {
        size_t bytes = round_up(count * sizeof(T), 256);
        T* r = reinterpret_cast<T*>(base + used);
        used += bytes;
        return r;
    }
    bool
    ok() const {
        return used <= size && (base != nullptr || used == 0);
    }
};

// ---- (distance, id) keys --------------------------------------------------------------------------
// A key orders by distance first and inner id second when compared as an unsigned 64-bit integer.
__host__ __device__ inline uint32_t
float_to_ordered(float f) {
#ifdef __HIP_DEVICE_COMPILE__
    uint32_t u = __float_as_uint(f);
#else
    uint32_t u;
    memcpy(&u, &f, 4);
#endif
    return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}

__host__ __device__ inline float
ordered_to_float(uint32_t u) {
    u ^= (u >> 31) ? 0x80000000u : 0xFFFFFFFFu;
#ifdef __HIP_DEVICE_COMPILE__
    return __uint_as_float(u);
#else
    float f;
    memcpy(&f, &u, 4);
    return f;
#endif
}

__host__ __device__ inline uint64_t
make_key(float dist, uint32_t id) {
    return (static_cast<uint64_t>(float_to_ordered(dist)) << 32) | id;
}

// Bit `id` of a deny mask (vsag_amd_search_options_t::deny_bits_dev); a null mask denies nothing.
__device__ inline bool
denied(const uint32_t* deny, uint64_t id) {
    return deny != nullptr && ((deny[id >> 5] >> (id & 31)) & 1U) != 0;
}

// The per-query bound a search starts from: nothing known, or the radius of a range search.
inline uint32_t
initial_bound(const vsag_amd_search_options_t* options) {
    return options != nullptr && options->use_radius ? float_to_ordered(options->radius) : 0xFFFFFFFFU;
}

}  // namespace vsag_amd
