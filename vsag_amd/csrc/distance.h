// Per-tile distance loops of every store kind: 64 codes (one per lane) against T queries at once.
//
// Every lane owns one code of the tile, so no cross-lane reduction is needed, and everything that is
// the same for all codes (per-dimension scales, the T processed queries) is read through the constant
// address space with wave-uniform addresses: the compiler turns those into s_load_dwordx16 and feeds
// the values to the VALU as SGPR operands, which costs no vector instruction and no LDS bandwidth.
//
// Reference arithmetic restated here (one query x one code each):
//   FP32   src/simd/kernels/compute_l2.h:27-76, compute_ip.h:38-90      (fp32_quantizer.cpp:164-188)
//   SQ8    src/simd/kernels/sq8_compute.h:44-137                        (scalar_quantizer.cpp:180-196)
//   SQ4    src/simd/generic.cpp:316-340, kernels/sq4_compute.h:21-95
//   SQ4U   src/simd/generic.cpp:406-422 + sq4_uniform_quantizer.cpp:166-201
//   SQ8U   src/simd/generic.cpp:424-431 + sq8_uniform_quantizer.cpp:141-170
//   RaBitQ src/simd/generic.cpp:832-872 + rabitq_quantizer.cpp:915-939,1775-1860
//   PQFS   src/simd/generic.cpp:902-921 (PQFastScanLookUp32) + pq_fastscan_quantizer.cpp:166-199
#pragma once

#include "common.h"

namespace vsag_amd {

typedef const float __attribute__((address_space(4))) * cfloat_p;
typedef const uint32_t __attribute__((address_space(4))) * cu32_p;

__device__ inline cfloat_p
as_const(const float* p) {
    return (cfloat_p)(uintptr_t)p;
}
__device__ inline cu32_p
as_const(const uint32_t* p) {
    return (cu32_p)(uintptr_t)p;
}

struct ScanArgs {
    const uint4* tiles;
    const uint32_t* meta;   // nmeta arrays of meta_stride words
    uint64_t meta_stride;
    const float* scale;     // sq8/sq4: per-dim scale, dpad floats
    const uint32_t* qtab;   // processed queries, qstride words each
    const float* qmeta;     // per-query scalars, qmeta_stride floats each
    uint32_t qstride;
    uint32_t qmeta_stride;
    uint32_t G;
    uint32_t dim;
    // multi-bit rabitq: granule j belongs to bit plane j / plane_granules ((j * plane_recip) >> 16 for the j in range)
    uint32_t planes, plane_granules, plane_recip;
    float f0, f1, f2;       // uniform kinds: lb, scalar_rate, lb*lb
};

// Tile rows are consumed in groups of GROUP granules so that the loads of the next group can be in flight
// while the current one is being multiplied (see TileStream below).

// Running sums of T queries against the code owned by this lane.
template <int KIND, int T>
struct Acc {
    float f[T];         // fp32 / sq8 / sq4; rabitq with fp32 queries: the sum under the bits of the current plane
    uint32_t lo[T];     // uniform kinds (and plane 0 of rabitq); multi-bit rabitq: the weighted sum of finished planes
                        // (float bits)
    uint32_t hi[T];     // sq4_uniform high nibbles (x16); rabitq plane 1
    uint32_t p2[T];     // rabitq plane 2
    uint32_t p3[T];     // rabitq plane 3
};

template <int KIND, int T>
__device__ inline void
acc_reset(Acc<KIND, T>& a) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
        a.f[t] = 0.0F;
        a.lo[t] = a.hi[t] = a.p2[t] = a.p3[t] = 0;
    }
}

// Wave-uniform row pointers of the T processed queries (constant address space -> scalar loads).
template <int T>
struct QueryRows {
    cu32_p row[T];
};

template <int T>
__device__ inline QueryRows<T>
query_rows(const ScanArgs& a, const uint32_t (&qidx)[T]) {
    QueryRows<T> r;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        r.row[t] = as_const(a.qtab + static_cast<size_t>(qidx[t]) * a.qstride);
    }
    return r;
}

// One granule (16 bytes of this lane's code, granule index j) against the T queries.
template <int KIND, int METRIC, int T>
__device__ __forceinline__ void
accumulate_granule(const ScanArgs& a, const QueryRows<T>& q, uint32_t j, uint4 c, Acc<KIND, T>& acc) {
    const uint32_t w[4] = {c.x, c.y, c.z, c.w};
    if constexpr (KIND == VSAG_AMD_KIND_FP32) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float x = __uint_as_float(w[e]);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                float qv = __uint_as_float(q.row[t][4 * j + e]);
                if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                    float d = x - qv;
                    acc.f[t] = fmaf(d, d, acc.f[t]);
                } else {
                    acc.f[t] = fmaf(x, qv, acc.f[t]);
                }
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
        // qtab row: L2 -> q[d] - lb[d];  IP -> q[d] * scale[d], qmeta[0] = sum q[d] * lb[d].
        cfloat_p sc = as_const(a.scale);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            float cf = static_cast<float>((w[e >> 2] >> (8 * (e & 3))) & 0xffU);
            if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                float y = cf * sc[16 * j + e];
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    float d = y - __uint_as_float(q.row[t][16 * j + e]);
                    acc.f[t] = fmaf(d, d, acc.f[t]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    acc.f[t] = fmaf(cf, __uint_as_float(q.row[t][16 * j + e]), acc.f[t]);
                }
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
        // Byte b of a code holds dim 2b in its low nibble and dim 2b+1 in its high nibble.
        cfloat_p sc = as_const(a.scale);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            uint32_t lo = w[m] & 0x0F0F0F0FU;
            uint32_t hi = (w[m] >> 4) & 0x0F0F0F0FU;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                uint32_t src = (e & 1) ? hi : lo;
                float cf = static_cast<float>((src >> (8 * (e >> 1))) & 0xffU);
                uint32_t d = 32 * j + 8 * m + e;
                if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                    float y = cf * sc[d];
#pragma unroll
                    for (int t = 0; t < T; ++t) {
                        float df = y - __uint_as_float(q.row[t][d]);
                        acc.f[t] = fmaf(df, df, acc.f[t]);
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < T; ++t) {
                        acc.f[t] = fmaf(cf, __uint_as_float(q.row[t][d]), acc.f[t]);
                    }
                }
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ4_UNIFORM) {
        // qtab row: per code dword {low nibbles, high nibbles}.  The code's high nibbles stay in place
        // (x16), so their products come out 16 times too large and are shifted back at the end.
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            uint32_t lo = w[m] & 0x0F0F0F0FU;
            uint32_t hi = w[m] & 0xF0F0F0F0U;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                acc.lo[t] = __builtin_amdgcn_udot4(lo, q.row[t][2 * (4 * j + m)], acc.lo[t], false);
                acc.hi[t] = __builtin_amdgcn_udot4(hi, q.row[t][2 * (4 * j + m) + 1], acc.hi[t], false);
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ8_UNIFORM) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                acc.lo[t] = __builtin_amdgcn_udot4(w[m], q.row[t][4 * j + m], acc.lo[t], false);
            }
        }
    } else if constexpr (KIND == kKindRabitqF32) {
        // qtab row: the rotated, centred, normalised query as fp32; a granule holds the bits of 128 dimensions.
        // Sum of the query values under set bits: a sign-extended one-bit extract is an all-ones / all-zeros
        // mask for the value.  Multi-bit codes (RaBitQFloatSplitCodeIP, generic.cpp:743-771: sum q[d] code[d]) are bit
        // planes of ceil(dim / 128) granules each, plane b first to last bit 0 to the top one: the sum under a plane
        // enters the total with weight 2^b when the plane ends.
        uint32_t plane = 0, jj = j;
        if (a.planes > 1) {
            plane = (j * a.plane_recip) >> 16;
            jj = j - plane * a.plane_granules;
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                uint32_t mask = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int32_t>(w[m]), e, 1));
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    acc.f[t] += __uint_as_float(mask & q.row[t][128 * jj + 32 * m + e]);
                }
            }
        }
        if (a.planes > 1 && jj + 1 == a.plane_granules) {
            const float weight = static_cast<float>(1U << plane);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                acc.lo[t] = __float_as_uint(fmaf(weight, acc.f[t], __uint_as_float(acc.lo[t])));
                acc.f[t] = 0.0F;
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_PQFS) {
        // qtab row: 16 table bytes per subspace.  A granule holds the centroid indices of 32 subspaces (byte b:
        // subspace 2 b in the low nibble, 2 b + 1 in the high one); every lane looks its own entries up, so these
        // are vector loads of one byte (all lanes inside the 16 bytes of one subspace: one memory line).
        typedef const uint8_t __attribute__((address_space(4))) * cu8_p;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t nib = (w[m] >> (4 * e)) & 15U;
                const uint32_t at = (32 * j + 8 * m + e) * 16 + nib;
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    acc.lo[t] += reinterpret_cast<cu8_p>(q.row[t])[at];
                }
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_RABITQ) {
        // qtab row: per code dword the four query bit planes.
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                cu32_p qp = q.row[t] + 4 * (4 * j + m);
                acc.lo[t] += __builtin_popcount(w[m] & qp[0]);
                acc.hi[t] += __builtin_popcount(w[m] & qp[1]);
                acc.p2[t] += __builtin_popcount(w[m] & qp[2]);
                acc.p3[t] += __builtin_popcount(w[m] & qp[3]);
            }
        }
    }
}

// Distances of the finished code (tile slot `slot`) to the T queries.
template <int KIND, int METRIC, int T>
__device__ __forceinline__ void
finish_distances(const ScanArgs& a, const uint32_t (&qidx)[T], uint64_t slot, const Acc<KIND, T>& acc,
                 float (&out)[T]) {
    if constexpr (KIND == VSAG_AMD_KIND_FP32) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
            out[t] = METRIC == VSAG_AMD_METRIC_L2 ? acc.f[t] : 1.0F - acc.f[t];
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ8 || KIND == VSAG_AMD_KIND_SQ4) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                out[t] = acc.f[t];
            } else {
                out[t] = 1.0F - (acc.f[t] + a.qmeta[static_cast<size_t>(qidx[t]) * a.qmeta_stride]);
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_SQ4_UNIFORM || KIND == VSAG_AMD_KIND_SQ8_UNIFORM) {
        float m0 = __uint_as_float(a.meta[slot]);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t ip = KIND == VSAG_AMD_KIND_SQ4_UNIFORM ? acc.lo[t] + (acc.hi[t] >> 4) : acc.lo[t];
            float result = static_cast<float>(static_cast<int32_t>(ip));
            float qm = a.qmeta[static_cast<size_t>(qidx[t]) * a.qmeta_stride];
            if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                // (float(norm_q) + float(norm_o) - 2 ip) * scalar_rate
                out[t] = (qm + m0 - 2 * result) * a.f1;
            } else {
                // 1 - (lb (sum_q + sum_o) + scalar_rate ip + lb^2)
                float r = a.f0 * (qm + m0) + a.f1 * result + a.f2;
                out[t] = 1 - r;
            }
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_PQFS) {
        // qmeta: {diff, lower} of the query's byte table; float(sum) / 255 * diff + lower, 1 - that for ip / cosine.
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float* qm = a.qmeta + static_cast<size_t>(qidx[t]) * a.qmeta_stride;
            const float v = static_cast<float>(static_cast<int32_t>(acc.lo[t])) / 255.0F * qm[0] + qm[1];
            out[t] = METRIC == VSAG_AMD_METRIC_L2 ? v : 1.0F - v;
        }
    } else if constexpr (KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32) {
        // qmeta, 4-bit queries: {2 delta/sqrt(d), 2 lb/sqrt(d), delta sum_q/sqrt(d), lb d/sqrt(d), ||Rq - c||, ||q||};
        // fp32 queries: {2/sqrt(d), -, sum_q/sqrt(d), -, ||Rq - c||, ||q||} (RaBitQFloatBinaryIP, generic.cpp:447-471:
        // +q/sqrt(d) under a set bit, -q/sqrt(d) under a clear one).
        float base_norm = __uint_as_float(a.meta[slot]);
        float base_error = __uint_as_float(a.meta[a.meta_stride + slot]);
        float base_sum = KIND == VSAG_AMD_KIND_RABITQ ? __uint_as_float(a.meta[2 * a.meta_stride + slot]) : 0.0F;
        float base_raw = METRIC == VSAG_AMD_METRIC_L2 ? 0.0F : __uint_as_float(a.meta[3 * a.meta_stride + slot]);
        if (static_cast<double>(fabsf(base_error)) < 1e-5) {
            base_error = (base_error >= 0) ? 1.0F : -1.0F;
        }
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float* qm = a.qmeta + static_cast<size_t>(qidx[t]) * a.qmeta_stride;
            float ip_bq;
            if constexpr (KIND == VSAG_AMD_KIND_RABITQ) {
                uint32_t ip = acc.lo[t] + (acc.hi[t] << 1) + (acc.p2[t] << 2) + (acc.p3[t] << 3);
                float p1 = qm[0] * static_cast<float>(ip);
                float p2 = qm[1] * base_sum;
                ip_bq = p1 + p2 - qm[2] - qm[3];
            } else if (a.planes > 1) {
                // ip_obar_q (rabitq_quantizer.cpp:256-267) of the plane-weighted sum; qm[1] = sum of the query values
                const float norm_code = __uint_as_float(a.meta[2 * a.meta_stride + slot]);
                const float c = 0.5F * static_cast<float>((1U << a.planes) - 1U);
                ip_bq = norm_code <= 0.0F ? 0.0F : (__uint_as_float(acc.lo[t]) - c * qm[1]) / norm_code;
            } else {
                ip_bq = qm[0] * acc.f[t] - qm[2];
            }
            float ip_est = ip_bq / base_error;
            float qn = qm[4];
            float e1 = base_norm * base_norm;
            float e2 = qn * qn;
            float e3 = -2 * base_norm * qn * ip_est;
            float result = e1 + e2 + e3;
            if constexpr (METRIC == VSAG_AMD_METRIC_IP) {
                float qr = qm[5];
                if (static_cast<double>(fabsf(qr)) < 1e-5 || static_cast<double>(fabsf(base_raw)) < 1e-5) {
                    result = 1;
                } else {
                    result = 1 - (qr * qr + base_raw * base_raw - result) * 0.5F;
                }
            } else if constexpr (METRIC == VSAG_AMD_METRIC_COSINE) {
                float qr = qm[5];
                if (static_cast<double>(fabsf(qr)) < 1e-5 || static_cast<double>(fabsf(base_raw)) < 1e-5) {
                    result = 1;
                } else {
                    result = 1 - (qr * qr + base_raw * base_raw - result) * 0.5F / (qr * base_raw);
                }
            }
            out[t] = result;
        }
    }
}

// The sequence of granule groups one wave walks: tiles first, first + stride, ... below end; inside a tile
// groups j0 = 0, GROUP, ...  `load` fetches a group into registers, `advance` steps to the next one.
// OVERLAP: when the granules of a tile are not a multiple of GROUP, the last group of a tile starts GROUP granules
// before the tile's end instead of running past it: it re-reads granules the previous group has just fetched
// (cache hits) rather than granules of the next tile (memory traffic), and only its new granules are consumed.
template <int GROUP, bool OVERLAP = false>
struct TileStream {
    const uint4* tiles;  // wave-uniform; a lane reads element `lane` of a 64-element granule row
    uint32_t lane;
    uint64_t tile, end, stride;
    uint32_t j0, G;

    __device__ inline bool
    valid() const {
        return tile < end;
    }
    // Always issues GROUP loads at fixed offsets from one row address, with no branch around any of them,
    // so that the consumer can wait for this group alone while the next one stays in flight.  A stream that
    // has run out reads `fallback` (any tile the caller knows to exist); the last group of a tile may run up
    // to GROUP - 1 granules past it, into the next tile or the slack that every tile buffer ends with
    // (kTileSlackBytes) -- those registers are never consumed.
    __device__ inline void
    load(uint4 (&regs)[GROUP], uint64_t fallback) const {
        const uint64_t t = tile < end ? tile : fallback;
        const uint4* tp = tiles + (t * G + first()) * kWave + lane;
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            regs[u] = tp[u * kWave];
        }
    }
    // Granule held by register 0 of the group at j0.
    __device__ inline uint32_t
    first() const {
        if constexpr (OVERLAP) {
            return G >= GROUP && j0 + GROUP > G ? G - GROUP : j0;
        }
        return j0;
    }
    __device__ inline void
    advance() {
        j0 += GROUP;
        if (j0 >= G) {
            j0 = 0;
            tile += stride;
        }
    }
};

}  // namespace vsag_amd
