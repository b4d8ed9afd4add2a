// Wave-level streaming top-k selector kept in LDS.
//
// One wavefront owns one selector per query it serves.  A selector is an array of S 64-bit keys
// (S a power of two, S >= k + 96): slots [0,k) hold the best keys found so far, slots [base, base+cnt), base =
// selector_base(S, k), hold pending candidates that passed the current threshold.  When an append would overflow
// the pending region, the wave flushes: the k best of everything end up in front, in ascending order, and
// keys[k-1] is the new threshold.  With k <= S / 2 (and S >= 256) the pending region is the upper half and a flush
// sorts only that half (downwards) and merges it into the sorted front -- half the compare-exchange steps of sorting
// the whole array, which is what the other selectors do.  No workgroup barrier is involved: only the owning
// wave touches a selector, and LDS operations of one wave complete in program order.
//
// This replaces the reference's per-query bounded max-heap (src/impl/heap/standard_heap.cpp:24-53,
// src/algorithm/ivf/flat_bucket_searcher.cpp:89-100): same k smallest distances, with ties ordered by
// inner id (the reference leaves the order of equal distances unspecified).
#pragma once

#include "common.h"

namespace vsag_amd {

__device__ inline void
wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ inline uint32_t
lane_id() {
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `mask` below this lane.
__device__ inline uint32_t
mask_rank(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

__device__ inline uint64_t
wave_uniform_u64(uint64_t v) {
    uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Selector size for a given k.
__host__ __device__ inline uint32_t
selector_slots(uint32_t k) {
    uint32_t s = 128;
    while (s < k + 96) {
        s <<= 1;
    }
    return s;
}

// First slot of the pending region.
__host__ __device__ inline uint32_t
selector_base(uint32_t S, uint32_t k) {
    return S >= 256 && 2 * k <= S ? S / 2 : k;
}

__device__ inline void
selector_init(uint64_t* keys, uint32_t S, uint32_t lane) {
    for (uint32_t i = lane; i < S; i += kWave) {
        keys[i] = kInfKey;
    }
    wave_lds_fence();
}

// Ascending bitonic sort of keys[0,S) by one wavefront.
__device__ inline void
wave_bitonic_sort(uint64_t* keys, uint32_t S, uint32_t lane) {
    for (uint32_t size = 2; size <= S; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t i = lane; i < (S >> 1); i += kWave) {
                uint32_t pos = 2 * i - (i & (stride - 1));
                uint64_t a = keys[pos];
                uint64_t b = keys[pos + stride];
                bool up = (pos & size) == 0;
                if ((a > b) == up) {
                    keys[pos] = b;
                    keys[pos + stride] = a;
                }
            }
            wave_lds_fence();
        }
    }
}

// One compare-exchange step of a bitonic network over keys[0, n): pairs `stride` apart, ascending where
// (pos & size) == 0 (size = 0: everywhere), descending elsewhere; `flip` turns the directions round.
__device__ inline void
wave_bitonic_step(uint64_t* keys, uint32_t n, uint32_t size, uint32_t stride, bool flip, uint32_t lane) {
    for (uint32_t i = lane; i < (n >> 1); i += kWave) {
        uint32_t pos = 2 * i - (i & (stride - 1));
        uint64_t a = keys[pos];
        uint64_t b = keys[pos + stride];
        bool up = ((pos & size) == 0) != flip;
        if ((a > b) == up) {
            keys[pos] = b;
            keys[pos + stride] = a;
        }
    }
    wave_lds_fence();
}

// Keeps the k best in front, in ascending order, and returns the new threshold key (wave-uniform).  keys[0, k) are in
// ascending order on entry (they are after selector_init and after every flush), cnt keys are pending.
__device__ inline uint64_t
selector_flush(uint64_t* keys, uint32_t S, uint32_t k, uint32_t cnt, uint32_t lane) {
    const uint32_t base = selector_base(S, k);
    for (uint32_t i = base + cnt + lane; i < S; i += kWave) {
        keys[i] = kInfKey;
    }
    wave_lds_fence();
    if (base == k) {
        wave_bitonic_sort(keys, S, lane);
        return wave_uniform_u64(keys[k - 1]);
    }
    // The front half is ascending (k keys, then kInfKey).  The pending half sorted downwards behind it makes the
    // whole array bitonic; one step across the halves leaves the smaller half in front, itself bitonic, and a
    // merge puts it in order.
    uint64_t* pending = keys + base;
    for (uint32_t size = 2; size <= base; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            wave_bitonic_step(pending, base, size == base ? 0 : size, stride, true, lane);
        }
    }
    for (uint32_t i = lane; i < base; i += kWave) {
        uint64_t a = keys[i];
        uint64_t b = keys[i + base];
        if (b < a) {
            keys[i] = b;
        }
    }
    wave_lds_fence();
    for (uint32_t stride = base >> 1; stride > 0; stride >>= 1) {
        wave_bitonic_step(keys, base, 0, stride, false, lane);
    }
    // Only the k best stay.
    for (uint32_t i = k + lane; i < base; i += kWave) {
        keys[i] = kInfKey;
    }
    wave_lds_fence();
    return wave_uniform_u64(keys[k - 1]);
}

// How many of keys[0,total) are real and have an ordered distance of at most `bound` (wave-uniform).
__device__ inline uint32_t
selector_count_admitted(const uint64_t* keys, uint32_t total, uint32_t bound, uint32_t lane) {
    uint32_t n = 0;
    for (uint32_t i0 = 0; i0 < total; i0 += kWave) {
        uint32_t i = i0 + lane;
        uint64_t key = i < total ? keys[i] : kInfKey;
        bool ok = key != kInfKey && static_cast<uint32_t>(key >> 32) <= bound;
        n += __popcll(__ballot(ok));
    }
    return n;
}

// Copies those keys to dst[0, count), in selector order.
__device__ inline void
selector_copy_admitted(const uint64_t* keys, uint32_t total, uint32_t bound, uint64_t* dst, uint32_t lane) {
    uint32_t n = 0;
    for (uint32_t i0 = 0; i0 < total; i0 += kWave) {
        uint32_t i = i0 + lane;
        uint64_t key = i < total ? keys[i] : kInfKey;
        bool ok = key != kInfKey && static_cast<uint32_t>(key >> 32) <= bound;
        uint64_t mask = __ballot(ok);
        if (ok) {
            dst[n + mask_rank(mask)] = key;
        }
        n += __popcll(mask);
    }
}

__device__ inline uint32_t
wave_min_u32(uint32_t v) {
    for (int off = 32; off > 0; off >>= 1) {
        uint32_t o = __shfl_xor(v, off);
        v = o < v ? o : v;
    }
    return __builtin_amdgcn_readfirstlane(v);
}

__device__ inline uint32_t
wave_max_u32(uint32_t v) {
    for (int off = 32; off > 0; off >>= 1) {
        uint32_t o = __shfl_xor(v, off);
        v = o > v ? o : v;
    }
    return __builtin_amdgcn_readfirstlane(v);
}

// Lowers *p to v if v is smaller; returns the smaller of v and the value seen (wave-uniform).  The atomic
// is skipped when a plain load already shows a value that is not larger.
__device__ inline uint32_t
lower_shared(uint32_t* p, uint32_t v, uint32_t lane) {
    uint32_t seen = __builtin_amdgcn_readfirstlane(__atomic_load_n(p, __ATOMIC_RELAXED));
    if (v < seen) {
        uint32_t old = lane == 0 ? atomicMin(p, v) : 0U;
        seen = __builtin_amdgcn_readfirstlane(old);
    }
    return seen < v ? seen : v;
}

}  // namespace vsag_amd
