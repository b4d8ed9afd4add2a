// Pre-selection for large query batches on a flat sq8 store of more than 128 dimensions, on the fp16 matrix cores.
//
// The int8 pass (prefilter_i8.hip) keeps a query's operands in registers, which ends at 128 dimensions; beyond that
// sq8 stores used the fp32 matrix cores (prefilter.hip, prefilter_kernel).  The contraction <b, c> of a code c (bytes
// 0..255) with the query b folded with the per-dimension scale (l2: b_d = (q_d - lb_d) scale_d, ip: b_d = q_d scale_d)
// does not need fp32 operands: a byte is exact in fp16, and b splits, after a power-of-two scaling per query, into two
// fp16 parts,
//
//      2^E b_d = hi_d + lo_d + r_d,     hi_d = fp16(2^E b_d),   lo_d = fp16(2^E b_d - hi_d),   |r_d| <= 2^-22 |2^E b_d|,
//
// whose products with a byte are exact in the fp32 accumulator of v_mfma_f32_32x32x16_f16, which runs at sixteen
// times the rate of the fp32 instruction: two of them per block of dimensions.  What the two parts miss (r_d, the
// rounding of b_d itself) is measured per query in double precision against the real product, times the largest code
// value; the accumulation of the matrix cores is allowed two roundings per instruction of the absolute sum.  Both go
// onto the query's threshold (h16_split_kernel), on top of the margin the fp32 pass already allows for the streaming
// kernel's own arithmetic (prefilter_tau_kernel).  Everything kept is rescored exactly, so the result equals the
// streaming scan's bit for bit.
//
// Work split as in prefilter_kernel: a workgroup of four waves multiplies 128 codes (two storage tiles) by 128 queries
// in stages of 64 dimensions; the stage sits in LDS as 16-byte slots of eight fp16 values, [block of eight dimensions]
// [row], the operand order of the instruction (lane % 32 = row, lane / 32 = which eight of sixteen dimensions).
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kH16M = 128;      // codes per workgroup tile
constexpr uint32_t kH16N = 128;      // queries per workgroup tile
constexpr uint32_t kH16Stage = 64;   // dimensions per stage: eight slots per row
constexpr uint32_t kH16Slots = kH16Stage / 8;
// fp16 parts of the query the matrix cores see: with one, what the second would carry goes onto the threshold instead
constexpr uint32_t kH16Planes = 1;

bool
prefilter_h16_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_SQ8 && s->nlist == 0 && s->dpad > 128 && s->pf_term != nullptr && s->pf_ymax != nullptr;
}

static uint64_t
h16_query_rows(uint64_t nq) {
    return round_up(nq, static_cast<uint64_t>(kH16N));
}
static uint32_t
h16_slots_per_row(const vsag_amd_store* s) {
    return round_up(s->dpad, kH16Stage) / 8;
}

// Scratch of the pass: the two planes, [plane][block of eight dimensions][query] of 16-byte slots, then a factor per query.
size_t
prefilter_h16_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    const uint64_t rows = h16_query_rows(nq);
    return 2ull * h16_slots_per_row(s) * rows * 16 + rows * sizeof(float);
}

struct H16SplitArgs {
    const float* qtab;   // processed queries (distance.h): l2 q - lb, ip q; zero beyond the dimension
    uint32_t qstride;
    uint32_t kdim;
    const float* scale;  // l2: per dimension; null: ones
    uint64_t nq, rows;   // rows: nq rounded up to whole workgroup tiles
    uint32_t slots;      // blocks of eight dimensions per row
    uint4* planes;
    float* factor;       // per query: dot_factor * 2^-E
    float* tau;          // per query, raised by the error of the split
    float dot_factor;
};

// One wave per query row (rows at or beyond nq: zeros).
__global__ void __launch_bounds__(64)
h16_split_kernel(H16SplitArgs p) {
    const uint64_t q = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const bool real = q < p.nq;
    const float* row = p.qtab + q * p.qstride;
    // the largest |b_d| and whether every entry is finite
    float amax = 0.0F;
    bool finite = true;
    if (real) {
        for (uint32_t d = lane; d < p.kdim; d += kWave) {
            const float b = static_cast<float>(static_cast<double>(row[d]) * (p.scale != nullptr ? static_cast<double>(p.scale[d]) : 1.0));
            finite = finite && b - b == 0.0F;
            amax = fmaxf(amax, fabsf(b));
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off));
    }
    finite = __ballot(!finite) == 0;
    const bool usable = real && finite && amax > 0.0F;
    // 2^E amax in [2^13, 2^14): hi stays far below the largest fp16, lo normal for all but the tiniest entries
    int e = 0;
    if (usable) {
        (void)frexpf(amax, &e);
        e = 14 - e;
        e = e > 120 ? 120 : e;  // (a tiny query keeps fewer bits rather than an infinite factor)
    }
    const float up = ldexpf(1.0F, e), down = ldexpf(1.0F, -e);
    double miss = 0.0, sum_abs = 0.0;
    for (uint32_t s = lane; s < p.slots; s += kWave) {
        halfx8 hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t d = 8 * s + i;
            double exact = 0.0;
            if (usable && d < p.kdim) {
                exact = static_cast<double>(row[d]) * (p.scale != nullptr ? static_cast<double>(p.scale[d]) : 1.0);
            }
            const float b = static_cast<float>(exact) * up;  // a power of two: exact
            const _Float16 h = static_cast<_Float16>(b);
            const _Float16 l = kH16Planes == 2 ? static_cast<_Float16>(b - static_cast<float>(h)) : static_cast<_Float16>(0.0F);
            hi[i] = h;
            lo[i] = l;
            const double kept = (static_cast<double>(static_cast<float>(h)) + static_cast<double>(static_cast<float>(l))) *
                                static_cast<double>(down);
            miss += fabs(kept - exact);
            sum_abs += fabs(kept);
        }
        p.planes[(0ull * p.slots + s) * p.rows + q] = __builtin_bit_cast(uint4, hi);
        p.planes[(1ull * p.slots + s) * p.rows + q] = __builtin_bit_cast(uint4, lo);
    }
    for (int off = 32; off > 0; off >>= 1) {
        miss += __shfl_xor(miss, off);
        sum_abs += __shfl_xor(sum_abs, off);
    }
    if (lane != 0) {
        return;
    }
    p.factor[q] = usable ? p.dot_factor * down : 0.0F;
    if (!real) {
        return;
    }
    if (!usable) {
        // NaN or infinite entries, or an all-zero query: every code is a candidate (the query overflows and streams)
        if (!finite) {
            p.tau[q] = 3.0e38F;
        }
        return;
    }
    // every code value lies in [0, 255]; two roundings of the running absolute sum per matrix instruction (sixteen
    // dimensions each, two instructions per block) and four for the closing operations
    const double roundings = 2.0 * (p.kdim / 8.0 + 4.0) * 5.9604644775390625e-8;
    const double extra = fabs(static_cast<double>(p.dot_factor)) * 255.0 * (miss + roundings * sum_abs);
    const float t = p.tau[q];
    const float raised = t + static_cast<float>(extra) * (1.0F + 1.0e-6F);
    p.tau[q] = raised < 3.0e38F ? raised : 3.0e38F;
}

struct PrefilterH16Args {
    const uint4* tiles;
    uint32_t G;
    uint64_t tile_begin, tile_end;
    uint64_t n;
    const uint4* planes;   // h16_split_kernel
    const float* factor;
    uint64_t nq, rows;
    uint32_t slots;        // blocks of eight dimensions per row (a multiple of kH16Slots)
    const float* term;     // per slot |y|^2
    float term_factor;     // 1 (l2) or 0 (ip)
    const float* tau;
    uint32_t* cand;
    uint32_t* cand_cnt;
    uint32_t cap;
    uint32_t groups;
};

struct H16Stage {
    uint4 a[kH16Slots][kH16M];
    uint4 b[kH16Planes][kH16Slots][kH16N];
};

// Sixteen code bytes as sixteen fp16 values (two slots).
__device__ inline void
h16_bytes_to_halves(uint4 g, uint4* lo8, uint4* hi8) {
    const uint32_t w[4] = {g.x, g.y, g.z, g.w};
    halfx8 out[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            out[h][i] = static_cast<_Float16>(static_cast<float>((w[2 * h + (i >> 2)] >> (8 * (i & 3))) & 0xffU));
        }
    }
    *lo8 = __builtin_bit_cast(uint4, out[0]);
    *hi8 = __builtin_bit_cast(uint4, out[1]);
}

__global__ void __launch_bounds__(256, 3)
prefilter_h16_kernel(PrefilterH16Args p) {
    __shared__ H16Stage stage;
    __shared__ float code_term[kH16M];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;   // which 64 codes of the tile
    const uint32_t wn = wave >> 1;  // which 64 queries of the tile
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * kH16N;  // below p.rows: the grid covers whole tiles of rows
    const uint32_t stages = p.slots / kH16Slots;
    const uint64_t span = p.tile_end - p.tile_begin;
    const uint64_t mtiles = (span + 1) / 2;

    float tau_n[2], fac_n[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint64_t q = q0 + wn * 64 + j * 32 + l32;
        tau_n[j] = q < p.nq ? p.tau[q] : -__builtin_inff();
        fac_n[j] = q < p.nq ? p.factor[q] : 0.0F;
    }

    // Code loader: thread (crow, cpart) takes granules 2 cpart and 2 cpart + 1 of the stage's four, for code crow.
    const uint32_t crow = tid & 127;
    const uint32_t cpart = tid >> 7;
    auto code_granule = [&](uint64_t mt, uint32_t j) __attribute__((always_inline)) {
        const uint64_t tile = p.tile_begin + 2 * mt + (crow >> 6);
        if (tile < p.tile_end && j < p.G) {
            return p.tiles[(tile * p.G + j) * kWave + (crow & 63)];
        }
        return make_uint4(0, 0, 0, 0);
    };
    // Query loader: 2 planes x 8 slots x 128 rows = 2048 slots per stage, eight per thread, consecutive threads on
    // consecutive rows (global and LDS alike).
    // (Separate variables, not an array: the array ended up in scratch memory.)
    uint4 rc0, rc1, rq0, rq1, rq2, rq3, rq4, rq5, rq6, rq7;
    auto query_slot = [&](uint32_t st, uint32_t r) __attribute__((always_inline)) {
        const uint32_t idx = tid + 256 * r;
        const uint32_t row = idx & 127, slot = (idx >> 7) & 7, plane = idx >> 10;
        return p.planes[(static_cast<uint64_t>(plane) * p.slots + st * kH16Slots + slot) * p.rows + q0 + row];
    };
    auto fetch = [&](uint64_t mt, uint32_t st) __attribute__((always_inline)) {
        rc0 = code_granule(mt, 4 * st + 2 * cpart);
        rc1 = code_granule(mt, 4 * st + 2 * cpart + 1);
        rq0 = query_slot(st, 0);
        rq1 = query_slot(st, 1);
        rq2 = query_slot(st, 2);
        rq3 = query_slot(st, 3);
        if constexpr (kH16Planes == 2) {
            rq4 = query_slot(st, 4);
            rq5 = query_slot(st, 5);
            rq6 = query_slot(st, 6);
            rq7 = query_slot(st, 7);
        }
    };
    auto park_codes = [&](uint32_t g, uint4 v) __attribute__((always_inline)) {
        uint4 lo8, hi8;
        h16_bytes_to_halves(v, &lo8, &hi8);
        stage.a[2 * (2 * cpart + g)][crow] = lo8;
        stage.a[2 * (2 * cpart + g) + 1][crow] = hi8;
    };
    auto park_query = [&](uint32_t r, uint4 v) __attribute__((always_inline)) {
        const uint32_t idx = tid + 256 * r;
        stage.b[idx >> 10][(idx >> 7) & 7][idx & 127] = v;
    };
    auto park = [&]() __attribute__((always_inline)) {
        park_codes(0, rc0);
        park_codes(1, rc1);
        park_query(0, rq0);
        park_query(1, rq1);
        park_query(2, rq2);
        park_query(3, rq3);
        if constexpr (kH16Planes == 2) {
            park_query(4, rq4);
            park_query(5, rq5);
            park_query(6, rq6);
            park_query(7, rq7);
        }
    };

    if (blockIdx.x < mtiles) {
        fetch(blockIdx.x, 0);
    }
    for (uint64_t mt = blockIdx.x; mt < mtiles; mt += p.groups) {
        floatx16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0.0F;
                }
            }
        }
        const uint64_t slot0 = (p.tile_begin + 2 * mt) * kWave;
        park();  // the stage is free: the previous tile's contraction ended with a barrier
        float my_term = 0.0F;
        if (tid < kH16M) {
            const uint64_t slot = slot0 + tid;
            const bool real = slot < p.n && p.tile_begin + 2 * mt + (tid >> 6) < p.tile_end;
            my_term = real ? p.term_factor * p.term[slot] : __builtin_inff();
        }
        __syncthreads();
        for (uint32_t st = 0; st < stages; ++st) {
            if (st + 1 < stages) {
                fetch(mt, st + 1);
            } else if (mt + p.groups < mtiles) {
                fetch(mt + p.groups, 0);
            }
#pragma unroll
            for (uint32_t ks = 0; ks < kH16Stage / 16; ++ks) {
                const uint32_t slot = 2 * ks + half;
                halfx8 a[2], bh[2], bl[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const uint4 va = stage.a[slot][wm * 64 + i * 32 + l32];
                    const uint4 vh = stage.b[0][slot][wn * 64 + i * 32 + l32];
                    const uint4 vl = kH16Planes == 2 ? stage.b[1][slot][wn * 64 + i * 32 + l32] : make_uint4(0, 0, 0, 0);
                    a[i] = __builtin_bit_cast(halfx8, va);
                    bh[i] = __builtin_bit_cast(halfx8, vh);
                    bl[i] = __builtin_bit_cast(halfx8, vl);
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], bh[j], acc[i][j], 0, 0, 0);
                        if constexpr (kH16Planes == 2) {
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], bl[j], acc[i][j], 0, 0, 0);
                        }
                    }
                }
            }
            if (st + 1 == stages && tid < kH16M) {
                // every wave is past this tile's first barrier, hence out of the previous tile's epilogue
                code_term[tid] = my_term;
            }
            __syncthreads();  // every wave has read the stage
            if (st + 1 < stages) {
                park();
                __syncthreads();
            }
        }
        // Nearly nothing passes: the verdicts of all 64 products of a lane branch-free, then the rare hits append.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t hits = 0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const float v = code_term[ml] + fac_n[j] * acc[i][j][e];
                    hits |= (v <= tau_n[j] ? 1U : 0U) << (16 * i + e);
                }
            }
            if (hits != 0) {
                const uint64_t q = q0 + wn * 64 + j * 32 + l32;
                while (hits != 0) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctz(hits));
                    hits &= hits - 1;
                    const uint32_t i = bit >> 4, e = bit & 15;
                    const uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const uint32_t pos = atomicAdd(&p.cand_cnt[q], 1U);
                    if (pos < p.cap) {
                        p.cand[q * p.cap + pos] = static_cast<uint32_t>(slot0 + ml);
                    }
                }
            }
        }
    }
}

// tau holds the thresholds of prefilter_tau_kernel for the store's bounds; scratch: prefilter_h16_scratch_bytes.
int
launch_prefilter_h16(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                     float* tau, uint8_t* scratch, uint32_t* cand, uint32_t* cand_cnt, uint32_t cap, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t rows = h16_query_rows(nq);
    const uint32_t slots = h16_slots_per_row(s);
    uint4* planes = reinterpret_cast<uint4*>(scratch);
    float* factor = reinterpret_cast<float*>(scratch + 2ull * slots * rows * 16);
    H16SplitArgs sp{};
    sp.qtab = reinterpret_cast<const float*>(a.qtab);
    sp.qstride = a.qstride;
    sp.kdim = s->dpad;
    sp.scale = l2 ? s->scale_dev : nullptr;
    sp.nq = nq;
    sp.rows = rows;
    sp.slots = slots;
    sp.planes = planes;
    sp.factor = factor;
    sp.tau = tau;
    sp.dot_factor = l2 ? -2.0F : -1.0F;
    hipLaunchKernelGGL(h16_split_kernel, dim3(static_cast<uint32_t>(rows)), dim3(kWave), 0, st, sp);
    PrefilterH16Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.tile_begin = tile_begin;
    p.tile_end = tile_end;
    p.n = s->n;
    p.planes = planes;
    p.factor = factor;
    p.nq = nq;
    p.rows = rows;
    p.slots = slots;
    p.term = s->pf_term;
    p.term_factor = l2 ? 1.0F : 0.0F;
    p.tau = tau;
    p.cand = cand;
    p.cand_cnt = cand_cnt;
    p.cap = cap;
    const uint64_t mtiles = (tile_end - tile_begin + 1) / 2;
    const uint64_t qtiles = rows / kH16N;
    // About six workgroups per compute unit (two rounds of the three that fit); a group walks every groups-th tile.
    uint64_t groups = div_up(static_cast<uint64_t>(device_cu_count()) * 6, qtiles);
    groups = std::max<uint64_t>(1, std::min<uint64_t>(groups, mtiles));
    p.groups = static_cast<uint32_t>(groups);
    timing_begin(st);
    hipLaunchKernelGGL(prefilter_h16_kernel, dim3(p.groups, static_cast<uint32_t>(qtiles)), dim3(256), 0, st, p);
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
