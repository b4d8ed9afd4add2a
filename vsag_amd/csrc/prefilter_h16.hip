// Pre-selection for large query batches on a flat sq8 store of more than 128 dimensions, on the fp16 matrix cores.
//
// The int8 pass (prefilter_i8.hip) keeps a query's operands in registers, which ends at 128 dimensions; beyond that
// sq8 stores used the fp32 matrix cores (prefilter.hip, prefilter_kernel).  The contraction <b, c> of a code c (bytes
// 0..255) with the query b folded with the per-dimension scale (l2: b_d = (q_d - lb_d) scale_d, ip: b_d = q_d scale_d)
// does not need fp32 operands: a byte is exact in fp16, and b is taken, after a power-of-two scaling per query, as
// its nearest fp16 value, hi_d = fp16(2^E b_d).  The products hi_d c_d are exact in the fp32 accumulator of
// v_mfma_f32_32x32x16_f16, which runs at sixteen times the rate of the fp32 instruction.  A pair is lost only if the
// matrix cores' product comes out too small (it comes off the distance, and the codes are not negative): what the
// fp16 values fall short of their b_d is summed per query in double precision, times the largest code value, and the
// accumulation is allowed two roundings per instruction of the absolute sum.  Both go onto the query's threshold
// (h16_split_kernel), next to what the streaming kernel's own fp32 arithmetic can be off by -- a multiple of the
// distance, not of |q| |y|, since no fp32 contraction stands between the test and the truth here.  (A second fp16
// part of the query would carry the 2^-12 the first misses; it doubles the matrix work and the LDS reads and saves
// less in rescoring than it costs.)  Everything kept is rescored exactly, so the result equals the streaming scan's
// bit for bit.
//
// Work split: a workgroup of four waves multiplies 256 codes (four storage tiles) by 128 queries in stages of 64
// dimensions, a wave 128 codes by 64 queries; the stage sits in LDS as 16-byte slots of eight fp16 values, [block of
// eight dimensions][row], the operand order of the instruction (lane % 32 = row, lane / 32 = which eight of sixteen
// dimensions).  The queries' fp16 values come from a table in the same slot-major order, so global loads and LDS writes
// are both contiguous.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kH16M = 256;      // codes per workgroup tile (= threads of a workgroup)
constexpr uint32_t kH16N = 128;      // queries per workgroup tile
constexpr uint32_t kH16Stage = 64;   // dimensions per stage: eight slots per row
constexpr uint32_t kH16Slots = kH16Stage / 8;


bool
prefilter_h16_supports(const vsag_amd_store* s) {
    return (s->kind == VSAG_AMD_KIND_SQ8 || s->kind == VSAG_AMD_KIND_SQ4) && s->nlist == 0 && s->dpad > 128 &&
           s->pf_term != nullptr && s->pf_ymax != nullptr;
}

static uint64_t
h16_query_rows(uint64_t nq) {
    return round_up(nq, static_cast<uint64_t>(kH16N));
}
static uint32_t
h16_slots_per_row(const vsag_amd_store* s) {
    return round_up(s->dpad, kH16Stage) / 8;
}

// Scratch of the pass: the queries' fp16 values, [block of eight dimensions][query] of 16-byte slots, then a factor per query.
size_t
prefilter_h16_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    const uint64_t rows = h16_query_rows(nq);
    return static_cast<size_t>(h16_slots_per_row(s)) * rows * 16 + rows * sizeof(float);
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
    float* tau;          // per query: keep a pair when term_factor |y|^2 + factor <hi, c> <= tau
    float dot_factor;
    float cmax;          // largest code value: 255 (sq8) or 15 (sq4)
    int is_l2;
    const float* qmeta;  // ip: sum q_d lb_d per query
    uint32_t qmeta_stride;
    const uint32_t* bound;      // per query, ordered-float bits; 0xFFFFFFFF = none yet
    const uint32_t* ymax_bits;  // largest |y| of the store (l2: scaled codes, ip: raw codes)
};

// One wave per query row (rows at or beyond nq: zeros).
__global__ void __launch_bounds__(64)
h16_split_kernel(H16SplitArgs p) {
    const uint64_t q = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const bool real = q < p.nq;
    const float* row = p.qtab + q * p.qstride;
    // the largest |b_d|, whether every entry is finite, and the query's |a|^2 and sum |a_d|
    float amax = 0.0F;
    bool finite = true;
    double a2 = 0.0, a1 = 0.0;
    if (real) {
        for (uint32_t d = lane; d < p.kdim; d += kWave) {
            const double a = static_cast<double>(row[d]);
            const float b = static_cast<float>(a * (p.scale != nullptr ? static_cast<double>(p.scale[d]) : 1.0));
            finite = finite && b - b == 0.0F;
            amax = fmaxf(amax, fabsf(b));
            a2 += a * a;
            a1 += fabs(a);
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off));
        a2 += __shfl_xor(a2, off);
        a1 += __shfl_xor(a1, off);
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
        halfx8 hi;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t d = 8 * s + i;
            double exact = 0.0;
            if (usable && d < p.kdim) {
                exact = static_cast<double>(row[d]) * (p.scale != nullptr ? static_cast<double>(p.scale[d]) : 1.0);
            }
            const float b = static_cast<float>(exact) * up;  // a power of two: exact
            const _Float16 h = static_cast<_Float16>(b);

            hi[i] = h;
            const double kept = static_cast<double>(static_cast<float>(h)) * static_cast<double>(down);
            // Only what makes the matrix cores' product too small can lose a pair (the codes are not negative, the
            // product comes off the distance): the parts of b_d the fp16 value falls short of.
            miss += exact > kept ? exact - kept : 0.0;
            sum_abs += fabs(kept);
        }
        p.planes[static_cast<uint64_t>(s) * p.rows + q] = __builtin_bit_cast(uint4, hi);
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
    const uint32_t bbits = p.bound[q];
    if (!finite || bbits == 0xFFFFFFFFU) {
        // no bound yet, or NaN / infinite entries: every code is a candidate (the query overflows and streams)
        p.tau[q] = 3.0e38F;
        return;
    }
    constexpr double kU = 5.9604644775390625e-8;  // 2^-24, the unit roundoff of fp32
    const double bd = static_cast<double>(ordered_to_float(bbits));
    const double ymax = static_cast<double>(__uint_as_float(*p.ymax_bits)) * (1.0 + 1.0e-6);
    const double dots = sqrt(a2) * ymax;  // |<a, y>| of any code
    double t;
    if (p.is_l2) {
        // The streaming kernel sums fl(fl(c s) - a)^2 in fp32: off from the real sum S by at most
        // 2u sum |y - a| |y| + (n + 2) u S <= 2u sqrt(S) |y| + (n + 2) u S to first order; twice that is allowed for.
        // |y|^2 per code is accumulated in double and rounded once.
        const double s_abs = fabs(bd);
        const double e_stream = 4.0 * kU * sqrt(s_abs) * ymax + 2.0 * (p.kdim + 4) * kU * s_abs;
        const double e_term = 2.0 * kU * ymax * ymax;
        // S = |a|^2 + |y|^2 - 2 <b, c>: the pair can matter when |y|^2 - 2 <b, c> <= bd - |a|^2 + errors
        t = bd - a2 + e_stream + e_term;
    } else {
        // dist = 1 - (fl(sum c a) + qmeta): the fp32 sum is off by at most n u sum |c a|, the two closing operations by u
        // of their results; twice that is allowed for.
        const double qm = p.qmeta != nullptr ? static_cast<double>(p.qmeta[q * p.qmeta_stride]) : 0.0;
        const double m = fmin(static_cast<double>(p.cmax) * a1, dots);
        const double e_stream = 2.0 * (p.kdim + 2) * kU * m + 4.0 * kU * (m + fabs(qm) + 1.0 + fabs(bd));
        t = bd - 1.0 + qm + e_stream;
    }
    // every code value lies in [0, cmax]: what the fp16 value misses of b_d, and two roundings of the running absolute
    // sum per matrix instruction (sixteen dimensions each) plus four for the closing operations
    const double roundings = 2.0 * (p.kdim / 16.0 + 4.0) * kU;
    const double extra = fabs(static_cast<double>(p.dot_factor)) * static_cast<double>(p.cmax) * (miss + roundings * sum_abs);
    // the test itself: fl(term + fl(factor acc)) against the threshold rounded to fp32
    const double e_test = 4.0 * kU * (ymax * ymax + 2.0 * dots + fabs(t) + extra);
    t += extra + e_test;
    const float tf = static_cast<float>(t);
    const float up1 = tf + fabsf(tf) * 1.2e-7F + 1.0e-37F;  // not below t after the rounding to fp32
    p.tau[q] = up1 < 3.0e38F ? up1 : 3.0e38F;
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
    uint4 b[kH16Slots][kH16N];
};

// Sixteen code bytes as sixteen fp16 values (two slots).  A byte b under the high byte 0x64 is the fp16 value
// 1024 + b (the spacing of fp16 is one from 1024 to 2048); taking 1024 off is exact.
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
__device__ inline uint32_t
h16_two_bytes(uint32_t w, uint32_t selector) {
    const uint32_t biased = __builtin_amdgcn_perm(0x64646464U, w, selector);
    const halfx2 v = __builtin_bit_cast(halfx2, biased) - halfx2{static_cast<_Float16>(1024.0F), static_cast<_Float16>(1024.0F)};
    return __builtin_bit_cast(uint32_t, v);
}
__device__ inline void
h16_bytes_to_halves(uint4 g, uint4* lo8, uint4* hi8) {
    // selector bytes 0..3 pick from w, 4..7 from the constant: (w.b0, 0x64, w.b1, 0x64) and (w.b2, 0x64, w.b3, 0x64)
    constexpr uint32_t kLow = 0x04010400U, kHigh = 0x04030402U;
    *lo8 = make_uint4(h16_two_bytes(g.x, kLow), h16_two_bytes(g.x, kHigh), h16_two_bytes(g.y, kLow), h16_two_bytes(g.y, kHigh));
    *hi8 = make_uint4(h16_two_bytes(g.z, kLow), h16_two_bytes(g.z, kHigh), h16_two_bytes(g.w, kLow), h16_two_bytes(g.w, kHigh));
}

// An sq4 granule (32 dimensions: byte b holds dimension 2 b in its low and 2 b + 1 in its high nibble) as 32 fp16
// values: word w of the granule is the slot of dimensions 8 w .. 8 w + 7.
__device__ inline uint4
h16_nibbles_to_halves(uint32_t w) {
    const uint32_t lo = w & 0x0F0F0F0FU, hi = (w >> 4) & 0x0F0F0F0FU;
    const halfx2 bias = halfx2{static_cast<_Float16>(1024.0F), static_cast<_Float16>(1024.0F)};
    uint32_t out[4];
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b) {
        // (low nibble of byte b, zero, high nibble of byte b, zero) under 0x64 in the high bytes
        const uint32_t pair = __builtin_amdgcn_perm(hi, lo, 0x0c040c00U + b * 0x00010001U) | 0x64006400U;
        out[b] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(halfx2, pair) - bias);
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
}

// A workgroup: 256 codes (four storage tiles) x 128 queries, a wave 128 codes x 64 queries (4 x 2 blocks of 32 x 32):
// 48 KiB of operands per stage from L2 for 2 M multiply-adds, 6 LDS reads per 8 matrix instructions.
template <int KIND>
__global__ void __launch_bounds__(256, 2)
prefilter_h16_kernel(PrefilterH16Args p) {
    __shared__ H16Stage stage;
    __shared__ float code_term[kH16M];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;   // which 128 codes of the tile
    const uint32_t wn = wave >> 1;  // which 64 queries of the tile
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * kH16N;  // below p.rows: the grid covers whole tiles of rows
    const uint32_t stages = p.slots / kH16Slots;
    const uint64_t span = p.tile_end - p.tile_begin;
    const uint64_t mtiles = (span + 3) / 4;

    float tau_n[2], fac_n[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint64_t q = q0 + wn * 64 + j * 32 + l32;
        tau_n[j] = q < p.nq ? p.tau[q] : -__builtin_inff();
        fac_n[j] = q < p.nq ? p.factor[q] : 0.0F;
    }

    // Code loader: thread t takes the stage's four granules of code t of the tile (storage tile t / 64, lane t % 64).
    auto code_granule = [&](uint64_t mt, uint32_t j) __attribute__((always_inline)) {
        const uint64_t tile = p.tile_begin + 4 * mt + (tid >> 6);
        if (tile < p.tile_end && j < p.G) {
            return p.tiles[(tile * p.G + j) * kWave + (tid & 63)];
        }
        return make_uint4(0, 0, 0, 0);
    };
    // Query loader: 8 slots x 128 rows per stage, four per thread, consecutive threads on consecutive rows (global and
    // LDS alike).  (Separate variables, not arrays: an array ended up in scratch memory.)
    uint4 rc0, rc1, rc2, rc3, rq0, rq1, rq2, rq3;
    auto query_slot = [&](uint32_t st, uint32_t r) __attribute__((always_inline)) {
        const uint32_t idx = tid + 256 * r;
        const uint32_t row = idx & 127, slot = idx >> 7;
        return p.planes[(static_cast<uint64_t>(st) * kH16Slots + slot) * p.rows + q0 + row];
    };
    auto fetch = [&](uint64_t mt, uint32_t st) __attribute__((always_inline)) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
            rc0 = code_granule(mt, 2 * st);
            rc1 = code_granule(mt, 2 * st + 1);
        } else {
            rc0 = code_granule(mt, 4 * st);
            rc1 = code_granule(mt, 4 * st + 1);
            rc2 = code_granule(mt, 4 * st + 2);
            rc3 = code_granule(mt, 4 * st + 3);
        }
        rq0 = query_slot(st, 0);
        rq1 = query_slot(st, 1);
        rq2 = query_slot(st, 2);
        rq3 = query_slot(st, 3);
    };
    auto park_codes = [&](uint32_t g, uint4 v) __attribute__((always_inline)) {
        uint4 lo8, hi8;
        h16_bytes_to_halves(v, &lo8, &hi8);
        stage.a[2 * g][tid] = lo8;
        stage.a[2 * g + 1][tid] = hi8;
    };
    auto park_query = [&](uint32_t r, uint4 v) __attribute__((always_inline)) {
        const uint32_t idx = tid + 256 * r;
        stage.b[idx >> 7][idx & 127] = v;
    };
    auto park = [&]() __attribute__((always_inline)) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
            stage.a[0][tid] = h16_nibbles_to_halves(rc0.x);
            stage.a[1][tid] = h16_nibbles_to_halves(rc0.y);
            stage.a[2][tid] = h16_nibbles_to_halves(rc0.z);
            stage.a[3][tid] = h16_nibbles_to_halves(rc0.w);
            stage.a[4][tid] = h16_nibbles_to_halves(rc1.x);
            stage.a[5][tid] = h16_nibbles_to_halves(rc1.y);
            stage.a[6][tid] = h16_nibbles_to_halves(rc1.z);
            stage.a[7][tid] = h16_nibbles_to_halves(rc1.w);
        } else {
            park_codes(0, rc0);
            park_codes(1, rc1);
            park_codes(2, rc2);
            park_codes(3, rc3);
        }
        park_query(0, rq0);
        park_query(1, rq1);
        park_query(2, rq2);
        park_query(3, rq3);
    };

    if (blockIdx.x < mtiles) {
        fetch(blockIdx.x, 0);
    }
    for (uint64_t mt = blockIdx.x; mt < mtiles; mt += p.groups) {
        floatx16 acc[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0.0F;
                }
            }
        }
        const uint64_t slot0 = (p.tile_begin + 4 * mt) * kWave;
        park();  // the stage is free: the previous tile's contraction ended with a barrier
        float my_term;
        {
            const uint64_t slot = slot0 + tid;
            const bool real = slot < p.n && p.tile_begin + 4 * mt + (tid >> 6) < p.tile_end;
            my_term = real ? p.term_factor * p.term[slot] : __builtin_inff();
        }
        __syncthreads();
        for (uint32_t st = 0; st < stages; ++st) {
            if (st + 1 < stages) {
                fetch(mt, st + 1);
            } else if (mt + p.groups < mtiles) {
                fetch(mt + p.groups, 0);
            }
#pragma unroll 2
            for (uint32_t ks = 0; ks < kH16Stage / 16; ++ks) {
                const uint32_t slot = 2 * ks + half;
                halfx8 a[4], b[2];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    a[i] = __builtin_bit_cast(halfx8, stage.a[slot][wm * 128 + i * 32 + l32]);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    b[j] = __builtin_bit_cast(halfx8, stage.b[slot][wn * 64 + j * 32 + l32]);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
                    }
                }
            }
            if (st + 1 == stages) {
                // every wave is past this tile's first barrier, hence out of the previous tile's epilogue
                code_term[tid] = my_term;
            }
            __syncthreads();  // every wave has read the stage
            if (st + 1 < stages) {
                park();
                __syncthreads();
            }
        }
        // Nearly nothing passes: the verdicts of all 128 products of a lane branch-free, then the rare hits append.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint64_t hits = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 128 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const float v = code_term[ml] + fac_n[j] * acc[i][j][e];
                    hits |= static_cast<uint64_t>(v <= tau_n[j] ? 1U : 0U) << (16 * i + e);
                }
            }
            if (hits != 0) {
                const uint64_t q = q0 + wn * 64 + j * 32 + l32;
                while (hits != 0) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctzll(hits));
                    hits &= hits - 1;
                    const uint32_t i = bit >> 4, e = bit & 15;
                    const uint32_t ml = wm * 128 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const uint32_t pos = atomicAdd(&p.cand_cnt[q], 1U);
                    if (pos < p.cap) {
                        p.cand[q * p.cap + pos] = static_cast<uint32_t>(slot0 + ml);
                    }
                }
            }
        }
    }
}

// tau: nq floats, written here from the queries' bounds; scratch: prefilter_h16_scratch_bytes.
int
launch_prefilter_h16(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                     const uint32_t* bound, float* tau, uint8_t* scratch, uint32_t* cand, uint32_t* cand_cnt, uint32_t cap,
                     hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t rows = h16_query_rows(nq);
    const uint32_t slots = h16_slots_per_row(s);
    uint4* planes = reinterpret_cast<uint4*>(scratch);
    float* factor = reinterpret_cast<float*>(scratch + static_cast<size_t>(slots) * rows * 16);
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
    sp.cmax = s->kind == VSAG_AMD_KIND_SQ4 ? 15.0F : 255.0F;
    sp.is_l2 = l2 ? 1 : 0;
    sp.qmeta = l2 ? nullptr : a.qmeta;
    sp.qmeta_stride = a.qmeta_stride;
    sp.bound = bound;
    sp.ymax_bits = s->pf_ymax;
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
    const uint64_t mtiles = (tile_end - tile_begin + 3) / 4;
    const uint64_t qtiles = rows / kH16N;
    // At most four workgroups per compute unit -- two rounds of the two that fit, and not one workgroup more: a few left
    // over for a third round would run it alone.  A group walks every groups-th tile.
    uint64_t groups = static_cast<uint64_t>(device_cu_count()) * 4 / qtiles;
    groups = std::max<uint64_t>(1, std::min<uint64_t>(groups, mtiles));
    p.groups = static_cast<uint32_t>(groups);
    timing_begin(st);
    if (s->kind == VSAG_AMD_KIND_SQ4) {
        hipLaunchKernelGGL(prefilter_h16_kernel<VSAG_AMD_KIND_SQ4>, dim3(p.groups, static_cast<uint32_t>(qtiles)), dim3(256), 0,
                           st, p);
    } else {
        hipLaunchKernelGGL(prefilter_h16_kernel<VSAG_AMD_KIND_SQ8>, dim3(p.groups, static_cast<uint32_t>(qtiles)), dim3(256), 0,
                           st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

// ---- posting lists -----------------------------------------------------------------------------------------------
// sq8 lists of more than 128 dimensions (no residual): the probe columns behind the first, grouped by list, as in
// ivf_f32_kernel (prefilter.hip) -- a work item is a chunk of a list's tiles x up to 128 of the pairs that probe it --
// with this file's contraction: the rows of the query side are fetched through the pair table.
constexpr uint32_t kIvfH16Pairs = kH16N;
constexpr uint32_t kIvfH16ChunkTiles = 32;  // as ivf_i8.hip: kIvfI8ChunkTiles, kIvfI8Chunks
constexpr uint32_t kIvfH16Chunks = 4;

bool
ivf_h16_supports(const vsag_amd_store* s) {
    return (s->kind == VSAG_AMD_KIND_SQ8 || s->kind == VSAG_AMD_KIND_SQ4) && s->nlist > 0 && s->dpad > 128 &&
           s->pf_term != nullptr && s->pf_ymax != nullptr &&
           s->ids_dev != nullptr && s->residual_centroids_dev == nullptr;
}
uint32_t
ivf_h16_pairs_per_item() {
    return kIvfH16Pairs;
}
// (one more row than queries: the row of a pair that does not exist is a row of zeros)
size_t
ivf_h16_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    return prefilter_h16_scratch_bytes(s, nq + 1);
}

struct IvfH16Args {
    const uint4* tiles;
    uint32_t G;
    const uint4* planes;
    const float* factor;
    uint64_t nq, rows;
    uint32_t slots;
    const float* term;
    float term_factor;
    const float* tau;
    const uint32_t* ids;            // per slot; the padding behind a list's last code holds no id and never passes
    const uint32_t* list_tile;      // per list: first tile, end tile
    const uint32_t* pair_off;       // pairs of list b: sorted_pair[pair_off[b] .. pair_off[b + 1])
    const uint32_t* item_off;       // items of list b: item_off[b] .. item_off[b + 1]
    const uint32_t* sorted_pair;    // query * nprobe + column
    uint32_t nlist, nprobe;
    uint32_t k;                     // records per private list
    uint64_t* partial;
    uint32_t* partial_cnt;          // zero before the launch; may end above k (overflow: the pair is scanned again)
    uint32_t* gate;                 // nq + 2 words as in ivf_i8.hip
};

template <int KIND>
__global__ void __launch_bounds__(256, 2)
ivf_h16_kernel(IvfH16Args p) {
    __shared__ H16Stage stage;
    __shared__ float code_term[kH16M];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;
    const uint32_t wn = wave >> 1;
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint32_t item = blockIdx.x;
    const cu32_p ioff = as_const(p.item_off);
    if (item >= ioff[p.nlist]) {
        return;  // the whole workgroup
    }
    uint32_t lo_b = 0, hi_b = p.nlist;
    while (hi_b - lo_b > 1) {
        const uint32_t mid = (lo_b + hi_b) >> 1;
        if (ioff[mid] <= item) {
            lo_b = mid;
        } else {
            hi_b = mid;
        }
    }
    const uint32_t b = lo_b;
    const uint32_t list_begin = as_const(p.list_tile)[2 * b], list_end = as_const(p.list_tile)[2 * b + 1];
    uint32_t chunks = (list_end - list_begin + kIvfH16ChunkTiles - 1) / kIvfH16ChunkTiles;
    chunks = chunks < kIvfH16Chunks ? chunks : kIvfH16Chunks;
    if (chunks == 0) {
        return;
    }
    const uint32_t per = (list_end - list_begin + chunks - 1) / chunks;
    const uint32_t chunk = (item - ioff[b]) % chunks;
    const uint32_t group = (item - ioff[b]) / chunks;
    uint32_t tile_begin = list_begin + chunk * per;
    tile_begin = tile_begin < list_end ? tile_begin : list_end;
    const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
    const uint32_t pbeg = as_const(p.pair_off)[b] + group * kIvfH16Pairs;
    const uint32_t pend = as_const(p.pair_off)[b + 1];
    const uint32_t mtiles = (tile_end - tile_begin + 3) / 4;
    if (mtiles == 0 || pbeg >= pend) {
        return;
    }
    const uint32_t stages = p.slots / kH16Slots;

    // The query rows of this item: thread t stages row t % 128 (slots t / 128 + 2 r), the query of pair pbeg + t % 128.
    uint64_t qsrc;
    {
        const uint32_t at = pbeg + (tid & 127);
        qsrc = at < pend ? as_const(p.sorted_pair)[at] / p.nprobe : p.nq;  // p.nq: no such pair, a row of zeros
    }
    float tau_n[2], fac_n[2];
    uint32_t pair_n[2], query_n[2];
    bool live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t at = pbeg + wn * 64 + j * 32 + l32;
        live[j] = at < pend;
        pair_n[j] = live[j] ? as_const(p.sorted_pair)[at] : 0U;
        query_n[j] = pair_n[j] / p.nprobe;
        tau_n[j] = live[j] ? p.tau[query_n[j]] : -__builtin_inff();
        fac_n[j] = live[j] ? p.factor[query_n[j]] : 0.0F;
    }

    auto code_granule = [&](uint32_t mt, uint32_t j) __attribute__((always_inline)) {
        const uint32_t tile = tile_begin + 4 * mt + (tid >> 6);
        if (tile < tile_end && j < p.G) {
            return p.tiles[(static_cast<uint64_t>(tile) * p.G + j) * kWave + (tid & 63)];
        }
        return make_uint4(0, 0, 0, 0);
    };
    uint4 rc0, rc1, rc2, rc3, rq0, rq1, rq2, rq3;
    auto query_slot = [&](uint32_t st, uint32_t r) __attribute__((always_inline)) {
        const uint32_t slot = (tid >> 7) + 2 * r;
        return p.planes[(static_cast<uint64_t>(st) * kH16Slots + slot) * p.rows + qsrc];
    };
    auto fetch = [&](uint32_t mt, uint32_t st) __attribute__((always_inline)) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
            rc0 = code_granule(mt, 2 * st);
            rc1 = code_granule(mt, 2 * st + 1);
        } else {
            rc0 = code_granule(mt, 4 * st);
            rc1 = code_granule(mt, 4 * st + 1);
            rc2 = code_granule(mt, 4 * st + 2);
            rc3 = code_granule(mt, 4 * st + 3);
        }
        rq0 = query_slot(st, 0);
        rq1 = query_slot(st, 1);
        rq2 = query_slot(st, 2);
        rq3 = query_slot(st, 3);
    };
    auto park_codes = [&](uint32_t g, uint4 v) __attribute__((always_inline)) {
        uint4 lo8, hi8;
        h16_bytes_to_halves(v, &lo8, &hi8);
        stage.a[2 * g][tid] = lo8;
        stage.a[2 * g + 1][tid] = hi8;
    };
    auto park = [&]() __attribute__((always_inline)) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
            stage.a[0][tid] = h16_nibbles_to_halves(rc0.x);
            stage.a[1][tid] = h16_nibbles_to_halves(rc0.y);
            stage.a[2][tid] = h16_nibbles_to_halves(rc0.z);
            stage.a[3][tid] = h16_nibbles_to_halves(rc0.w);
            stage.a[4][tid] = h16_nibbles_to_halves(rc1.x);
            stage.a[5][tid] = h16_nibbles_to_halves(rc1.y);
            stage.a[6][tid] = h16_nibbles_to_halves(rc1.z);
            stage.a[7][tid] = h16_nibbles_to_halves(rc1.w);
        } else {
            park_codes(0, rc0);
            park_codes(1, rc1);
            park_codes(2, rc2);
            park_codes(3, rc3);
        }
        stage.b[(tid >> 7) + 0][tid & 127] = rq0;
        stage.b[(tid >> 7) + 2][tid & 127] = rq1;
        stage.b[(tid >> 7) + 4][tid & 127] = rq2;
        stage.b[(tid >> 7) + 6][tid & 127] = rq3;
    };

    fetch(0, 0);
    for (uint32_t mt = 0; mt < mtiles; ++mt) {
        floatx16 acc[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0.0F;
                }
            }
        }
        const uint64_t slot0 = (static_cast<uint64_t>(tile_begin) + 4 * mt) * kWave;
        park();
        float my_term;
        {
            // (a padding slot is all zeros: under inner product that is a good distance)
            const bool real = tile_begin + 4 * mt + (tid >> 6) < tile_end && p.ids[slot0 + tid] != VSAG_AMD_INVALID_ID;
            my_term = real ? p.term_factor * p.term[slot0 + tid] : __builtin_inff();
        }
        __syncthreads();
        for (uint32_t st = 0; st < stages; ++st) {
            if (st + 1 < stages) {
                fetch(mt, st + 1);
            } else if (mt + 1 < mtiles) {
                fetch(mt + 1, 0);
            }
#pragma unroll 2
            for (uint32_t ks = 0; ks < kH16Stage / 16; ++ks) {
                const uint32_t slot = 2 * ks + half;
                halfx8 a[4], bq[2];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    a[i] = __builtin_bit_cast(halfx8, stage.a[slot][wm * 128 + i * 32 + l32]);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    bq[j] = __builtin_bit_cast(halfx8, stage.b[slot][wn * 64 + j * 32 + l32]);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], bq[j], acc[i][j], 0, 0, 0);
                    }
                }
            }
            if (st + 1 == stages) {
                code_term[tid] = my_term;
            }
            __syncthreads();
            if (st + 1 < stages) {
                park();
                __syncthreads();
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint64_t hits = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 128 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const float v = code_term[ml] + fac_n[j] * acc[i][j][e];
                    hits |= static_cast<uint64_t>(v <= tau_n[j] ? 1U : 0U) << (16 * i + e);
                }
            }
            if (hits != 0 && live[j]) {
                const uint64_t list = (static_cast<uint64_t>(pair_n[j]) * kIvfH16Chunks + chunk) * 2 + wm;
                while (hits != 0) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctzll(hits));
                    hits &= hits - 1;
                    const uint32_t i = bit >> 4, e = bit & 15;
                    const uint32_t ml = wm * 128 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const uint32_t pos = atomicAdd(&p.partial_cnt[list], 1U);
                    if (pos < p.k) {
                        p.partial[list * p.k + pos] = slot0 + ml;
                    } else if (pos == p.k) {
                        if (atomicExch(&p.gate[query_n[j]], 1U) == 0U) {
                            atomicAdd(&p.gate[p.nq], 1U);
                        }
                    }
                }
            }
        }
    }
}

// Thresholds and fp16 query values from the bounds (tau: nq floats; scratch: ivf_h16_scratch_bytes), then the
// candidates of probe columns [p0, nprobe) grouped by list (pair_off, sorted_pair; item_off counted with
// ivf_h16_pairs_per_item() pairs per item) into the private lists (pair * 8 + chunk * 2 + half of the code tile) of
// kcand records in `partial`; partial_cnt zero before.  gate: nq + 2 words.
int
launch_ivf_h16(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
               const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, float* tau,
               uint8_t* scratch, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t rows = h16_query_rows(nq + 1);
    const uint32_t slots = h16_slots_per_row(s);
    uint4* planes = reinterpret_cast<uint4*>(scratch);
    float* factor = reinterpret_cast<float*>(scratch + static_cast<size_t>(slots) * rows * 16);
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
    sp.cmax = s->kind == VSAG_AMD_KIND_SQ4 ? 15.0F : 255.0F;
    sp.is_l2 = l2 ? 1 : 0;
    sp.qmeta = l2 ? nullptr : a.qmeta;
    sp.qmeta_stride = a.qmeta_stride;
    sp.bound = bound;
    sp.ymax_bits = s->pf_ymax;
    hipLaunchKernelGGL(h16_split_kernel, dim3(static_cast<uint32_t>(rows)), dim3(kWave), 0, st, sp);
    IvfH16Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.planes = planes;
    p.factor = factor;
    p.nq = nq;
    p.rows = rows;
    p.slots = slots;
    p.term = s->pf_term;
    p.term_factor = l2 ? 1.0F : 0.0F;
    p.tau = tau;
    p.ids = s->ids_dev;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.k = kcand;
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kIvfH16Pairs)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfH16Chunks;
    timing_begin(st);
    if (s->kind == VSAG_AMD_KIND_SQ4) {
        hipLaunchKernelGGL(ivf_h16_kernel<VSAG_AMD_KIND_SQ4>, dim3(static_cast<uint32_t>(max_items)), dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL(ivf_h16_kernel<VSAG_AMD_KIND_SQ8>, dim3(static_cast<uint32_t>(max_items)), dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
