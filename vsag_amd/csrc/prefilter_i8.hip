// Pre-selection for large query batches on a flat sq8 (or sq8_uniform, see UniformQuantizeArgs; or sq4, see
// QuantizeArgs::nibbles) store of at most 128 dimensions, on the int8 matrix cores.
//
// The streaming distance of an sq8 code is a function of <b, c>: c the code bytes (0..255), b the query folded
// with the per-dimension scale (l2: b_d = (q_d - lb_d) scale_d, ip: b_d = q_d scale_d).  Each query row b is split
// once, in double precision, into two int8 planes and a remainder,
//
//      b_d = s2 (256 h_d + l_d) + e_d,      h_d, l_d in [-128, 127],   s2 = max|b| / (127 * 256),
//
// so that <b, c> = s2 (256 <h, c> + <l, c>) + <e, c>.  The two integer products come out of
// v_mfma_i32_32x32x32_i8 exactly; the remainder is bounded rigorously per query by 255 max(sum of positive e_d,
// sum of negative e_d), because every c_d lies in [0, 255].  The matrix cores take signed bytes: the staged codes
// are c_d - 128 (one xor per word), and 128 sum_d (256 h_d + l_d) moves into the per-query threshold.
//
// A (query, code) pair is kept when its distance, lowered by every error term (the remainder above, the rounding
// of the streaming kernel's own fp32 arithmetic, the rounding of the per-code |y|^2 and of the test itself), does
// not exceed the query's bound.  The kept pairs are rescored exactly (rescore_kernel, prefilter.hip), so the
// result equals the streaming scan's bit for bit.
//
// Work split: a workgroup is four waves; each wave keeps the operands of 64 queries (both planes, 64 registers)
// for the whole kernel and meets every 64-code storage tile the workgroup walks, which is staged in LDS in the
// tile's own granule-major order -- that order is the operand order of the matrix instruction (lane % 32 = code,
// lane / 32 = which 16 of the 32 dimensions of a step), so staging is a plain copy.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kI8Dims = 128;       // dimensions the kernel covers (eight granules, four matrix steps)
constexpr uint32_t kI8QueryBytes = 256;  // two planes of 128 bytes per query
constexpr uint32_t kI8Group = 256;       // queries per workgroup

struct QuantizeArgs {
    const float* qtab;  // processed queries (distance.h): l2 q - lb, ip q * scale; zero beyond the dimension
    uint32_t qstride;
    uint32_t kdim;        // <= 128
    const float* scale;   // l2: per-dimension scale folded into b; ip: null
    const float* qmeta;   // ip: sum q_d lb_d per query
    uint32_t qmeta_stride;
    int is_l2;
    // sq4: the codes hold two 4-bit values per byte (byte b of a 32-dimension granule: dimension 2 b low, 2 b + 1
    // high).  They are staged as they are (0..15 needs no shift to fit a signed byte), a granule as its low and its high
    // nibbles, so operand position 16 g + p (staged granule g, byte p) is dimension 32 (g / 2) + 2 p + g % 2, and
    // the terms that make up for the shift by 128 of byte codes fall away.
    int nibbles;
    const uint32_t* bound;      // per query, ordered-float bits; 0xFFFFFFFF = none yet
    const uint32_t* ymax_bits;  // largest |y| of the store (l2: scaled codes, ip: raw codes)
    uint64_t nq, nq_pad;
    uint8_t* q8;     // nq_pad x 256 bytes
    float* amax;     // l2: per query max |b| (rounded up; 0 for queries that take no part), written by query_amax_kernel
    float* ginv;     // l2: per group of kI8Group queries, 1 / (2 s2) of the scale the group shares (0: no scale)
    uint32_t* tau;   // smallest T that passes (int32); l2: T is the matrix product minus the code's integer term
    // Per query, what the threshold needs besides the bound (kI8Scalars doubles: q_err, w, a2, b1, s2, usable): kept
    // so that a later level of the same call only redoes the threshold (retau_queries_i8_kernel).
    double* scal;
};

constexpr uint32_t kI8Scalars = 6;

// The threshold of one query against its current bound from the scalars of its quantization: see
// quantize_queries_i8_kernel for what they are.
__device__ inline uint32_t
query_tau_i8(const QuantizeArgs& p, uint64_t q, double q_err, double w, double a2, double b1, double s2, bool usable) {
    const uint32_t bbits = p.bound[q];
    if (bbits == 0xFFFFFFFFU || !usable) {
        // No bound yet, a query with NaN / infinite entries, or (l2) a group of all-zero queries, whose test would
        // have no scale: everything is a candidate (and the query will overflow into the streaming kernel).
        return 0x80000000U;
    }
    constexpr double kU = 5.9604644775390625e-8;  // 2^-24, the unit roundoff of fp32
    const double bd = static_cast<double>(ordered_to_float(bbits));
    const double ymax = static_cast<double>(__uint_as_float(*p.ymax_bits)) * (1.0 + 1.0e-6);
    const double shift = p.nibbles ? 0.0 : 128.0;  // the codes are staged as c - shift
    const double cmax = p.nibbles ? 15.0 : 255.0;  // largest code value
    if (p.is_l2) {
        // The streaming kernel sums fl(fl(c s) - a)^2 in fp32: off from the real sum S by at most
        // 2u sum |y - a| |y| + (n + 2) u S <= 2u sqrt(S) |y| + (n + 2) u S to first order; twice that is allowed for.
        const double s_abs = fabs(bd);
        const double e_stream = 4.0 * kU * sqrt(s_abs) * ymax + 2.0 * (p.kdim + 4) * kU * s_abs;
        // |y|^2 per code is accumulated in double and rounded once.
        const double e_term = 2.0 * kU * ymax * ymax;
        // dist = a2 + |y|^2 - 2 s2 (M + shift w) - 2 <e, c>, M the integer the matrix cores deliver: the pair can matter
        // when |y|^2 - 2 s2 M <= t_real, i.e. M >= |y|^2 / (2 s2) - t_real / (2 s2).
        const double t_real = bd - a2 + 2.0 * shift * s2 * w + 2.0 * q_err + e_stream + e_term;
        // The kernel subtracts I = rn(fl(|y|^2 inv)) from M, inv = fl(1 / (2 s2)) (ginv): I differs from the real
        // |y|^2 / (2 s2) by at most a half plus two fp32 roundings of a value of at most ymax^2 / (2 s2); the kernel
        // clamps I from above only, which admits more.  So M - I >= floor(-t_real / (2 s2) - that - 1) keeps every
        // pair the real test keeps.
        const double x_max = ymax * ymax / (2.0 * s2);
        const double x = floor(-t_real / (2.0 * s2) - 0.5 - 4.0 * kU * x_max - 1.0);
        const int32_t ti = x >= 2147483647.0 ? 0x7FFFFFFF : (x <= -2147483648.0 ? static_cast<int32_t>(0x80000000U)
                                                                                 : static_cast<int32_t>(x));
        return static_cast<uint32_t>(ti);
    }
    // dist = 1 - (fl(sum c a) + qmeta): the fp32 sum is off by at most n u sum |c a|, the two closing
    // operations by u of their results; twice that is allowed for.
    const double qm = p.qmeta != nullptr ? static_cast<double>(p.qmeta[q * p.qmeta_stride]) : 0.0;
    const double m = fmin(cmax * b1, sqrt(a2) * ymax * (1.0 + 1.0e-6));
    const double e_stream = 2.0 * (p.kdim + 2) * kU * m + 4.0 * kU * (m + fabs(qm) + 1.0 + fabs(bd));
    // 1 - qm - s2 (T + shift w) - <e, c> <= bd   <=>   T >= -(bd - 1 + qm + errors) / s2 - shift w.
    const double rhs = bd - 1.0 + qm + q_err + e_stream;
    int32_t ti;
    if (s2 > 0.0) {
        const double x = floor(-rhs / s2 - shift * w) - 2.0;
        ti = x >= 2147483647.0 ? 0x7FFFFFFF : (x <= -2147483648.0 ? static_cast<int32_t>(0x80000000U)
                                                                  : static_cast<int32_t>(x));
    } else {
        ti = rhs >= 0.0 ? static_cast<int32_t>(0x80000000U) : 0x7FFFFFFF;
    }
    return static_cast<uint32_t>(ti);
}

__device__ inline double
wave_sum_f64(double v) {
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off);
    }
    return v;
}

__device__ inline double
wave_max_f64(double v) {
    for (int off = 32; off > 0; off >>= 1) {
        double o = __shfl_xor(v, off);
        v = o > v ? o : v;
    }
    return v;
}

// The l2 test compares the matrix product with a per-code integer (|y|^2 / 2 s2, see prefilter_i8_kernel), so the
// kI8Group queries that meet a code in one workgroup must share the scale s2: it is taken from the largest |b| of the
// group.  A query much smaller than its group's largest loses resolution (more candidates, never a wrong result).
// One wave per query: amax[q] = max_d |b_d|, rounded up to a float; 0 for padding rows and rows with NaN / infinite
// entries (they pass everything anyway and must not blow up the scale of their group).
__global__ void __launch_bounds__(64)
query_amax_kernel(QuantizeArgs p) {
    const uint64_t q = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    double m = 0.0;
    if (q < p.nq) {
        const float* row = p.qtab + q * p.qstride;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const uint32_t d = lane + 64 * r;
            if (d < p.kdim) {
                const double a = static_cast<double>(row[d]);
                const double b = fabs(p.scale != nullptr ? a * static_cast<double>(p.scale[d]) : a);
                m = b > m || !(b < 1.0e300) ? b : m;
            }
        }
    }
    // NaN wins the reduction so that a bad row is seen as such.
    for (int off = 32; off > 0; off >>= 1) {
        const double o = __shfl_xor(m, off);
        m = o > m || !(o < 1.0e300) ? o : m;
    }
    if (lane == 0) {
        float f = 0.0F;
        if (m < 1.0e30) {
            f = static_cast<float>(m);
            f = static_cast<double>(f) < m ? __uint_as_float(__float_as_uint(f) + 1U) : f;  // m > 0 here: next float up
        }
        p.amax[q] = f;
    }
}

// One wave per query; lane l owns dimensions l and l + 64.
__global__ void __launch_bounds__(64)
quantize_queries_i8_kernel(QuantizeArgs p) {
    const uint64_t q = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    uint8_t* out = p.q8 + q * kI8QueryBytes;
    // l2: the scale of the whole group.
    double gmax = 0.0;
    if (p.is_l2) {
        const uint64_t g0 = q / kI8Group * kI8Group;
        float m = 0.0F;
#pragma unroll
        for (int r = 0; r < static_cast<int>(kI8Group / kWave); ++r) {
            m = fmaxf(m, p.amax[g0 + lane + kWave * r]);
        }
        for (int off = 32; off > 0; off >>= 1) {
            m = fmaxf(m, __shfl_xor(m, off));
        }
        gmax = static_cast<double>(m);
        if (q == g0 && lane == 0) {
            // 1 / (2 s2) as the kernel multiplies the code terms with it.
            p.ginv[q / kI8Group] = gmax > 0.0 ? static_cast<float>(127.0 * 256.0 / (2.0 * gmax)) : 0.0F;
        }
    }
    if (q >= p.nq) {
        // Padding rows: zero operands and a threshold nothing meets.
        out[lane] = 0;
        out[64 + lane] = 0;
        out[128 + lane] = 0;
        out[192 + lane] = 0;
        if (lane == 0) {
            p.tau[q] = 0x7FFFFFFFU;
        }
        return;
    }
    const float* row = p.qtab + q * p.qstride;
    double a[2], b[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint32_t d = lane + 64 * r;
        a[r] = d < p.kdim ? static_cast<double>(row[d]) : 0.0;
        // The product of two floats is exact in double.
        b[r] = p.scale != nullptr && d < p.kdim ? a[r] * static_cast<double>(p.scale[d]) : a[r];
    }
    const double own_max = wave_max_f64(fmax(fabs(b[0]), fabs(b[1])));
    // A row with NaN / infinite entries is not part of its group's maximum; it keeps zero operands and passes
    // everything (below).
    const bool bad_row = !(own_max < 1.0e30);
    const double amax = p.is_l2 ? (bad_row ? 0.0 : gmax) : own_max;
    const double s1 = amax / 127.0;
    const double s2 = s1 / 256.0;
    double e_pos = 0.0, e_neg = 0.0, w = 0.0;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        double h = 0.0, l = 0.0;
        if (amax > 0.0) {
            h = fmin(fmax(rint(b[r] / s1), -127.0), 127.0);
            l = fmin(fmax(rint((b[r] - s1 * h) / s2), -128.0), 127.0);
        }
        const double whole = 256.0 * h + l;  // an integer below 2^16: exact
        const double e = b[r] - s2 * whole;
        e_pos += e > 0.0 ? e : 0.0;
        e_neg += e < 0.0 ? -e : 0.0;
        w += whole;
        const uint32_t d = lane + 64 * r;
        const uint32_t at = p.nibbles ? 16 * (2 * (d >> 5) + (d & 1U)) + ((d & 31U) >> 1) : d;
        out[at] = static_cast<uint8_t>(static_cast<int8_t>(h));
        out[128 + at] = static_cast<uint8_t>(static_cast<int8_t>(l));
    }
    e_pos = wave_sum_f64(e_pos);
    e_neg = wave_sum_f64(e_neg);
    w = wave_sum_f64(w);  // exact: integers
    const double a2 = wave_sum_f64(a[0] * a[0] + a[1] * a[1]);
    const double b1 = wave_sum_f64(fabs(b[0]) + fabs(b[1]));
    if (lane != 0) {
        return;
    }
    // |<e, c>| for any code, plus the rounding of the double arithmetic above.
    const double cmax = p.nibbles ? 15.0 : 255.0;
    const double q_err = cmax * fmax(e_pos, e_neg) + 1.0e-12 * cmax * b1;
    const bool usable = (b1 < 1.0e300) && (a2 < 1.0e300) && !bad_row && !(p.is_l2 && !(s2 > 0.0));
    if (p.scal != nullptr) {
        double* keep = p.scal + q * kI8Scalars;
        keep[0] = q_err;
        keep[1] = w;
        keep[2] = a2;
        keep[3] = b1;
        keep[4] = s2;
        keep[5] = usable ? 1.0 : 0.0;
    }
    p.tau[q] = query_tau_i8(p, q, q_err, w, a2, b1, s2, usable);
}

// A later level of the same call: the planes stand, only the bound has moved.  One thread per query; merged_dists
// (may be null) holds the k best distances of everything before this level, whose k-th lowers the bound first.
__global__ void __launch_bounds__(256)
retau_queries_i8_kernel(QuantizeArgs p, const float* merged_dists, uint32_t k, uint32_t* bound) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q >= p.nq) {
        return;
    }
    if (merged_dists != nullptr) {
        const float kth = merged_dists[q * k + k - 1];
        if (kth < __builtin_inff()) {
            const uint32_t o = float_to_ordered(kth);
            if (o < bound[q]) {
                bound[q] = o;
            }
        }
    }
    const double* keep = p.scal + q * kI8Scalars;
    p.tau[q] = query_tau_i8(p, q, keep[0], keep[1], keep[2], keep[3], keep[4], keep[5] != 0.0);
}

// sq8_uniform (and, with 4-bit values, sq4_uniform) stores: the query is a row of bytes itself (its uniform code, 0..255), so the product with the code is
// an integer the matrix cores deliver exactly.  A byte q splits as 256 h + l with h in {0, 1} and l in [-128, 127];
// with the codes staged as c - 128 the kernel's T = 256 H + L is <code, query> - 128 sum(query).  The streaming
// distance is a short fp32 expression of that integer and two scalars (distance.h, finish_distances):
//      l2:       ((norm_q + norm_o) - 2 ip) rate            ip/cosine:  1 - (lb (sum_q + sum_o) + rate ip + lb^2)
// so "distance <= bound" becomes the kernel's test fma(T, u, term_o) <= tau with (u, term_o) = (-2, norm_o) or
// (-rate, -lb sum_o), and tau carrying the bound, the query's scalars and every rounding of both forms.
struct UniformQuantizeArgs {
    const uint32_t* qtab;  // the queries' uniform codes, qstride words each
    uint32_t qstride;
    uint32_t kdim;         // <= 128
    const float* qmeta;    // per query: norm (l2) or sum (ip, cosine) of its code
    uint32_t qmeta_stride;
    int is_l2;
    int nibbles;           // sq4_uniform: qtab holds, per code dword, a word of low-nibble and one of high-nibble values
    float lb, rate, lb2;
    const uint32_t* bound;
    uint64_t nq, nq_pad;
    uint8_t* q8;
    float* u;
    uint32_t* tau;
    double* scal;  // per query kI8Scalars doubles, the first holds the sum of the query's values (see QuantizeArgs)
};

// The threshold of one query of a uniform kind against its current bound; sum = the sum of the query's values.
__device__ inline uint32_t
uniform_tau_i8(const UniformQuantizeArgs& p, uint64_t q, double sum) {
    const uint32_t bbits = p.bound[q];
    const double rate = static_cast<double>(p.rate);
    if (bbits == 0xFFFFFFFFU) {
        return __float_as_uint(3.0e38F);  // no bound yet: everything is a candidate
    }
    constexpr double kU = 5.9604644775390625e-8;  // 2^-24
    const double bd = static_cast<double>(ordered_to_float(bbits));
    const double qm = static_cast<double>(p.qmeta[q * p.qmeta_stride]);
    const double cmax = p.nibbles ? 15.0 : 255.0;      // largest code value
    const double shift = p.nibbles ? 0.0 : 128.0;      // the codes are staged as c - shift
    const double ip_max = cmax * sum;                  // <code, query> of any code
    const double t_max = 128.0 * 256.0 * p.kdim;       // |T| of any code
    const double m_max = p.is_l2 ? cmax * cmax * p.kdim : cmax * p.kdim;  // norm_o, sum_o of any code
    double t;
    if (p.is_l2) {
        // Streaming: fl(fl(fl(qm + m) - 2 R) rate), R the integer as a float (exact below 2^24).  The two sums round
        // by at most u of their magnitude each, the product by u of itself.
        if (!(rate > 0.0)) {
            return __float_as_uint(3.0e38F);
        }
        const double reach = fabs(qm) + m_max + 2.0 * ip_max;
        const double x_max = bd / rate * (1.0 + 4.0 * kU) + 4.0 * kU * reach;  // what qm + m - 2 ip may reach
        // qm + m - 2 (T + shift sum) <= x_max   <=>   m - 2 T <= x_max - qm + 2 shift sum
        t = x_max - qm + 2.0 * shift * sum;
        // The test itself: fl(m - 2 T) in one fma against the rounded threshold.
        t += 4.0 * kU * (m_max + 2.0 * t_max + fabs(t));
    } else {
        // Streaming: r = fl(fl(fl(lb fl(qm + m)) + fl(rate R)) + lb2), distance fl(1 - r).
        const double lb = fabs(static_cast<double>(p.lb)), lb2 = fabs(static_cast<double>(p.lb2));
        const double reach = lb * (fabs(qm) + m_max) + rate * ip_max + lb2 + 1.0 + fabs(bd);
        const double e_stream = 8.0 * kU * reach;
        // 1 - lb (qm + m) - rate (T + shift sum) - lb2 <= bd + e
        //     <=>   -rate T - lb m <= bd + e - 1 + lb qm + shift rate sum + lb2
        t = bd + e_stream - 1.0 + static_cast<double>(p.lb) * qm + shift * rate * sum + static_cast<double>(p.lb2);
        // term_o = fl(-lb m) and the fma of the test.
        t += 4.0 * kU * (2.0 * lb * m_max + rate * t_max + fabs(t));
    }
    return __float_as_uint(t < 3.0e38 ? (t > -3.0e38 ? static_cast<float>(t) : -3.0e38F) : 3.0e38F);
}

// One wave per query; lane l owns dimensions l and l + 64.
__global__ void __launch_bounds__(64)
quantize_uniform_i8_kernel(UniformQuantizeArgs p) {
    const uint64_t q = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    uint8_t* out = p.q8 + q * kI8QueryBytes;
    if (q >= p.nq) {
        out[lane] = 0;
        out[64 + lane] = 0;
        out[128 + lane] = 0;
        out[192 + lane] = 0;
        if (lane == 0) {
            p.u[q] = 0.0F;
            p.tau[q] = __float_as_uint(-__builtin_inff());
        }
        return;
    }
    const uint32_t* row = p.qtab + q * p.qstride;
    double sum = 0.0;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint32_t d = lane + 64 * r;  // operand position: staged granule d / 16, byte d % 16
        uint32_t v = 0;
        if (p.nibbles) {
            // Staged granule g holds the low (g even) or high (g odd) nibbles of code bytes 16 (g / 2) ...
            const uint32_t g = d >> 4, b = 16 * (g >> 1) + (d & 15);
            v = 2 * b + (g & 1) < p.kdim ? (row[2 * (b >> 2) + (g & 1)] >> (8 * (b & 3))) & 255U : 0U;
        } else {
            v = d < p.kdim ? (row[d >> 2] >> (8 * (d & 3))) & 255U : 0U;
        }
        const uint32_t h = v >> 7;
        out[d] = static_cast<uint8_t>(h);
        out[128 + d] = static_cast<uint8_t>(v - 256U * h);  // the low byte of the two's complement of v - 256 h
        sum += static_cast<double>(v);
    }
    sum = wave_sum_f64(sum);  // exact: integers
    if (lane != 0) {
        return;
    }
    p.u[q] = p.is_l2 ? -2.0F : -p.rate;
    if (p.scal != nullptr) {
        p.scal[q * kI8Scalars] = sum;
    }
    p.tau[q] = uniform_tau_i8(p, q, sum);
}

// A later level of the same call (see retau_queries_i8_kernel).
__global__ void __launch_bounds__(256)
retau_uniform_i8_kernel(UniformQuantizeArgs p, const float* merged_dists, uint32_t k, uint32_t* bound) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q >= p.nq) {
        return;
    }
    if (merged_dists != nullptr) {
        const float kth = merged_dists[q * k + k - 1];
        if (kth < __builtin_inff()) {
            const uint32_t o = float_to_ordered(kth);
            if (o < bound[q]) {
                bound[q] = o;
            }
        }
    }
    p.tau[q] = uniform_tau_i8(p, q, p.scal[q * kI8Scalars]);
}

struct PrefilterI8Args {
    const uint4* tiles;
    uint32_t G;
    uint64_t tile_begin, tile_end;
    uint64_t n;
    const uint4* q8;      // [query][plane][granule]
    uint64_t nq;
    const float* term;    // per slot: |y|^2 (sq8 l2) or the uniform kinds' term
    const float* u;       // per query (fma test)
    const float* ginv;    // per group of kI8Group queries: 1 / (2 s2) (integer test with a code term)
    const uint32_t* tau;  // per query
    // Candidates go to private lists: list (group, lane / 32) of a query belongs to one lane of one wave for the
    // whole kernel, so appending needs no atomic and nobody waits for one.
    uint32_t* cand;       // [query][2 groups][sub_cap]
    uint32_t* cand_cnt;   // [query][2 groups]; a count above sub_cap means the list overflowed
    uint32_t sub_cap;
    uint32_t groups;      // stage g of the span (kI8StageTiles tiles) is walked by group g % groups
    uint32_t qgroups;     // groups of kI8Group queries; the grid is groups x qgroups workgroups in one dimension
};

constexpr int kI8StageTiles = 2;  // storage tiles per LDS stage (one barrier per stage)

// How a (query, code) pair is judged from M = 256 H + L, the two matrix products:
//   kI8TestFma      fl(fl(M) u_q + term_o) <= tau_q in fp32 (the uniform kinds: term_o and u_q from their formulas);
//   kI8TestInt      M >= tau_q (sq8 inner product: the per-code part of the distance is in M already);
//   kI8TestIntTerm  M - I_o >= tau_q (sq8 l2) with I_o = rn(term_o / 2 s2) the code's |y|^2 in units of the product.
//                   -I_o is what the accumulator of L starts from, so the matrix pipe does the subtraction and the
//                   test costs what the plain integer test costs.
constexpr int kI8TestFma = 0;
constexpr int kI8TestInt = 1;
constexpr int kI8TestIntTerm = 2;

struct I8Stage {
    uint4 codes[kI8StageTiles][8 * kWave];  // granule-major, as in the store; bytes are c - 128
    float term[kI8StageTiles][kWave];       // kI8TestIntTerm: the bits of the int32 -I_o
};

// Largest code term in units of the product; beyond it the term is clamped (which only admits more).
constexpr float kI8TermClamp = 1073741824.0F;  // 2^30

// NIBBLE: the codes hold two 4-bit values per byte (sq4_uniform, at most four granules per code): a granule is staged
// as two, its low nibbles and its high nibbles, as they are (0..15 needs no shift to fit a signed byte).
template <int TEST, bool NIBBLE = false>
__global__ void __launch_bounds__(256, 2)
prefilter_i8_kernel(PrefilterI8Args p) {
    __shared__ I8Stage stage[2];
    constexpr bool kTerm = TEST != kI8TestInt;  // a per-code term takes part in the test
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    // Workgroups are handed to the eight XCDs (each with its own L2) in turn.  All query groups that walk the same
    // stages are made neighbours on one XCD, so that a tile is fetched into that L2 once and found there by the
    // others: the fabric carries the codes once instead of once per query group.
    uint32_t gx, gy;
    if ((p.groups & 7U) == 0) {
        const uint32_t xcd = blockIdx.x & 7U, local = blockIdx.x >> 3;
        gy = local % p.qgroups;
        gx = (local / p.qgroups) * 8 + xcd;
    } else {
        gx = blockIdx.x % p.groups;
        gy = blockIdx.x / p.groups;
    }
    const uint64_t q_base = (static_cast<uint64_t>(gy) * 4 + wave) * kWave;
    const bool active = q_base < p.nq;  // the query table is padded to whole workgroups
    const uint64_t span = p.tile_end - p.tile_begin;
    const uint64_t nstages = (span + kI8StageTiles - 1) / kI8StageTiles;

    // Query operands: block j = queries q_base + 32 j + lane % 32; step s = dimensions 32 s + 16 (lane / 32) ...
    intx4 qh[2][4], ql[2][4];
    float uq[2];
    uint32_t tau[2];
    uint32_t ncand[2] = {0, 0};
    uint32_t* my_list[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint64_t q = q_base + 32 * j + l32;
        const uint4* rowp = p.q8 + q * (kI8QueryBytes / 16);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint4 hv = rowp[2 * s + half];
            const uint4 lv = rowp[8 + 2 * s + half];
            qh[j][s] = intx4{static_cast<int>(hv.x), static_cast<int>(hv.y), static_cast<int>(hv.z),
                             static_cast<int>(hv.w)};
            ql[j][s] = intx4{static_cast<int>(lv.x), static_cast<int>(lv.y), static_cast<int>(lv.z),
                             static_cast<int>(lv.w)};
        }
        uq[j] = TEST == kI8TestFma ? p.u[q] : 0.0F;
        tau[j] = p.tau[q];
        my_list[j] = p.cand + ((q < p.nq ? q : 0) * 2 * p.groups + 2 * gx + half) * p.sub_cap;
    }
    const float ginv = TEST == kI8TestIntTerm ? p.ginv[gy] : 0.0F;

    // Staging: wave w copies granules w and w + 4 of each tile of the stage, a lane per code.
    uint4 regs[kI8StageTiles][2];
    float my_term[kI8StageTiles];
    auto fetch = [&](uint64_t sg) {
#pragma unroll
        for (int tt = 0; tt < kI8StageTiles; ++tt) {
            const uint64_t tile = p.tile_begin + sg * kI8StageTiles + tt;
            const bool real = tile < p.tile_end;
#pragma unroll
            for (int r = 0; r < (NIBBLE ? 1 : 2); ++r) {
                const uint32_t j = wave + 4 * r;
                // Raw bytes; they turn into c - 128 when parked, so that nothing waits for the load here.
                const uint32_t none = NIBBLE ? 0U : 0x80808080U;
                regs[tt][r] = make_uint4(none, none, none, none);
                if (real && j < p.G) {
                    regs[tt][r] = p.tiles[(tile * p.G + j) * kWave + lane];
                }
            }
            if constexpr (kTerm) {
                my_term[tt] = 0.0F;
                if (wave == 0) {
                    const uint64_t slot = tile * kWave + lane;
                    my_term[tt] = real && slot < p.n ? p.term[slot] : __builtin_inff();
                }
            }
        }
    };
    auto park = [&](I8Stage& st) {
#pragma unroll
        for (int tt = 0; tt < kI8StageTiles; ++tt) {
            if constexpr (NIBBLE) {
                const uint4 v = regs[tt][0];
                const uint32_t m = 0x0F0F0F0FU;
                st.codes[tt][(2 * wave) * kWave + lane] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
                st.codes[tt][(2 * wave + 1) * kWave + lane] =
                    make_uint4((v.x >> 4) & m, (v.y >> 4) & m, (v.z >> 4) & m, (v.w >> 4) & m);
            } else {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const uint4 v = regs[tt][r];
                    st.codes[tt][(wave + 4 * r) * kWave + lane] =
                        make_uint4(v.x ^ 0x80808080U, v.y ^ 0x80808080U, v.z ^ 0x80808080U, v.w ^ 0x80808080U);
                }
            }
            if constexpr (kTerm) {
                if (wave == 0) {
                    if constexpr (TEST == kI8TestIntTerm) {
                        // -I_o, I_o = rn(term / 2 s2) clamped from above (a slot without a code: the clamp itself,
                        // such a slot is never appended).  A term of NaN compares false and converts to 0.
                        const float x = my_term[tt] * ginv;
                        const int32_t io = x >= kI8TermClamp ? static_cast<int32_t>(kI8TermClamp) : __float2int_rn(x);
                        st.term[tt][lane] = __int_as_float(-io);
                    } else {
                        st.term[tt][lane] = my_term[tt];
                    }
                }
            }
        }
    };

    // A stage is a run of 32 x 32 blocks: block b = (tile b / 4 of the stage, codes 32 ((b / 2) % 2) ..., queries
    // 32 (b % 2) ...).  The matrix instructions of block b + 1 are issued among the verdict instructions of block b,
    // so that the matrix pipe and the vector ALU of the wave run side by side.
    constexpr int kBlocks = 4 * kI8StageTiles;
    // The grid never has more columns than there are stages, so the first stage exists.  Fetching it without a
    // condition also lets every load issued so far (the query operands) complete here, once, instead of being
    // waited for inside the loop, where that wait would hold up the prefetch of the next stage.
    uint64_t sg = gx;
    fetch(sg);
    park(stage[0]);
    __syncthreads();
    uint32_t cur = 0;
    for (; sg < nstages; sg += p.groups) {
        const uint64_t sn = sg + p.groups;
        if (sn < nstages) {
            fetch(sn);
        }
        if (active) {
            const I8Stage& st = stage[cur];
            const uint64_t slot0 = (p.tile_begin + sg * kI8StageTiles) * kWave;
            intx16 hi[2], lo[2];  // two sets: one being filled, one being judged
            // Row r of the stage = codes 32 (r % 2) ... of its tile r / 2; blocks 2 r and 2 r + 1 are its two query
            // halves.  Code operands and terms of a row are read from LDS one block before their first use
            // (two register sets each), so that no matrix instruction and no verdict waits for LDS.
            intx4 av[2][4];
            float tm[2][16];
            auto read_row = [&](int r) {
                const int tt = r >> 1, i = r & 1;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint4 c = st.codes[tt][(2 * s + half) * kWave + 32 * i + l32];
                    av[r & 1][s] = intx4{static_cast<int>(c.x), static_cast<int>(c.y), static_cast<int>(c.z),
                                         static_cast<int>(c.w)};
                }
                if constexpr (kTerm) {
                    // Element e of a lane is code 32 i + 8 (e / 4) + 4 (lane / 32) + e % 4 of the tile.
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const float4 v = *reinterpret_cast<const float4*>(&st.term[tt][32 * i + 8 * g + 4 * half]);
                        tm[r & 1][4 * g] = v.x;
                        tm[r & 1][4 * g + 1] = v.y;
                        tm[r & 1][4 * g + 2] = v.z;
                        tm[r & 1][4 * g + 3] = v.w;
                    }
                }
            };
            auto multiply = [&](int b, intx16& h, intx16& l) {
                const int r = b >> 1, j = b & 1;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    h[e] = 0;
                    // The low product starts from minus the code's integer term: M - I_o comes out of the matrix pipe.
                    l[e] = TEST == kI8TestIntTerm ? __float_as_int(tm[r & 1][e]) : 0;
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    h = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[r & 1][s], qh[j][s], h, 0, 0, 0);
                    l = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[r & 1][s], ql[j][s], l, 0, 0, 0);
                }
            };
            // The quantity of element e that is compared with the query's threshold.
            auto judged_int = [&](int b, int e) { return (hi[b & 1][e] << 8) + lo[b & 1][e]; };
            auto judged_fma = [&](int b, int e) {
                return fmaf(static_cast<float>(judged_int(b, e)), uq[b & 1], tm[(b >> 1) & 1][e]);
            };
            read_row(0);
            multiply(0, hi[0], lo[0]);
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
                const int r = b >> 1, j = b & 1;
                constexpr int kDsReads = kTerm ? 8 : 4;
                const bool reads = j == 0 && b + 2 < kBlocks;
                if (reads) {
                    read_row(r + 1);
                }
                if (b + 1 < kBlocks) {
                    multiply(b + 1, hi[(b + 1) & 1], lo[(b + 1) & 1]);
                }
                // Nearly nothing passes.  The sixteen elements of a lane are reduced to their best one with
                // three-operand max / min instructions (none of them writing a scalar register) -- four at a time, so
                // that a block with a hit finds it group by group -- and one compare decides whether the block needs a
                // second look.
                bool hit;
                float gbest_f[4];
                int32_t gbest_i[4];
                if constexpr (TEST == kI8TestFma) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        gbest_f[g] = fminf(fminf(fminf(judged_fma(b, 4 * g), judged_fma(b, 4 * g + 1)), judged_fma(b, 4 * g + 2)),
                                           judged_fma(b, 4 * g + 3));
                    }
                    hit = fminf(fminf(fminf(gbest_f[0], gbest_f[1]), gbest_f[2]), gbest_f[3]) <= __uint_as_float(tau[j]);
                } else {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        gbest_i[g] = max(max(max(judged_int(b, 4 * g), judged_int(b, 4 * g + 1)), judged_int(b, 4 * g + 2)),
                                         judged_int(b, 4 * g + 3));
                    }
                    hit = max(max(max(gbest_i[0], gbest_i[1]), gbest_i[2]), gbest_i[3]) >= static_cast<int32_t>(tau[j]);
                }
                const uint64_t any = __ballot(hit);
                if (b + 1 < kBlocks) {
                    // The LDS reads first; then one matrix instruction (32 cycles of the pipe) at a time, each
                    // followed by its share of the verdict instructions.
                    if (reads) {
                        __builtin_amdgcn_sched_group_barrier(0x100, kDsReads, 0);
                    }
#pragma unroll
                    for (int m = 0; m < 8; ++m) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, TEST == kI8TestFma ? 8 : 4, 0);
                    }
                }
                if (any != 0) {
                    // Some lane has an element that passes: find the groups of four with a hit, judge their elements
                    // one by one (the accumulators of this block are not touched before the next block has been
                    // judged) and let the lanes under each element's mask append.
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        bool ghit;
                        if constexpr (TEST == kI8TestFma) {
                            ghit = gbest_f[g] <= __uint_as_float(tau[j]);
                        } else {
                            ghit = gbest_i[g] >= static_cast<int32_t>(tau[j]);
                        }
                        if (__ballot(ghit) == 0) {
                            continue;
                        }
#pragma unroll
                        for (int e = 4 * g; e < 4 * g + 4; ++e) {
                            bool pass;
                            if constexpr (TEST == kI8TestFma) {
                                pass = judged_fma(b, e) <= __uint_as_float(tau[j]);
                            } else {
                                pass = judged_int(b, e) >= static_cast<int32_t>(tau[j]);
                            }
                            if (__ballot(pass) != 0) {
                                const uint64_t slot = slot0 + 32 * r + 8 * (e >> 2) + 4 * half + (e & 3);
                                if (pass && slot < p.n) {
                                    if (ncand[j] < p.sub_cap) {
                                        my_list[j][ncand[j]] = static_cast<uint32_t>(slot);
                                    }
                                    ++ncand[j];
                                }
                            }
                        }
                    }
                }
            }
        }
        if (sn < nstages) {
            park(stage[cur ^ 1]);
        }
        __syncthreads();  // the next stage is complete, and every wave is done with this one
        cur ^= 1;
    }
    if (active) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint64_t q = q_base + 32 * j + l32;
            if (q < p.nq) {
                p.cand_cnt[q * 2 * p.groups + 2 * gx + half] = ncand[j];
            }
        }
    }
}

bool
prefilter_i8_supports(const vsag_amd_store* s) {
    if (s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4) {
        return s->nlist == 0 && s->pf_term != nullptr && s->dpad <= kI8Dims && s->G <= 4;
    }
    return (s->kind == VSAG_AMD_KIND_SQ8 || s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) && s->nlist == 0 && s->pf_term != nullptr &&
           s->dpad <= kI8Dims && s->G <= 8;
}

size_t prefilter_i8_query_bytes(uint64_t nq);
size_t prefilter_i8_scalar_floats(uint64_t nq);

// ---- sq8 (and, NIBBLE, sq4) posting lists against large batches --------------------------------------------------------------------
// The same two-plane test over the (query, list) pairs of an ivf search that the streaming kernel has already given a
// bound (the probe columns behind the nearest list, see ivf_i8.hip for the work split this kernel shares: a
// workgroup = a chunk of a list's tiles x up to 256 of the pairs that probe the list, four waves of 64 pairs).  The
// queries of a workgroup are whatever queries probe the list, so they cannot share a scale by groups of neighbours:
// the whole batch shares one (spread_amax_kernel), and 1 / (2 s2) is one number.  What passes is recorded as a tile
// slot in the private list of (pair, chunk, lane / 32) -- the lists the streaming kernel's partial results use -- and
// turned into a (distance, id) key by ivf_rescore_kernel (prefilter.hip).
constexpr uint32_t kIvfSq8Pairs = 256;
constexpr uint32_t kIvfSq8ChunkTiles = 32;  // as ivf_i8.hip: kIvfI8ChunkTiles, kIvfI8Chunks
constexpr uint32_t kIvfSq8Chunks = 4;

// amax[q] = the largest amax of the batch, for every row (one workgroup).
__global__ void __launch_bounds__(1024)
spread_amax_kernel(float* amax, uint64_t n) {
    __shared__ float part[16];
    float m = 0.0F;
    for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) {
        m = fmaxf(m, amax[i]);
    }
    for (int off = 32; off > 0; off >>= 1) {
        m = fmaxf(m, __shfl_xor(m, off));
    }
    if ((threadIdx.x & 63) == 0) {
        part[threadIdx.x >> 6] = m;
    }
    __syncthreads();
    m = 0.0F;
    for (uint32_t w = 0; w < blockDim.x / kWave; ++w) {
        m = fmaxf(m, part[w]);
    }
    for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) {
        amax[i] = m;
    }
}

struct IvfSq8Args {
    const uint4* tiles;
    uint32_t G;
    const float* term;           // per slot |y|^2 (l2)
    const uint32_t* list_tile;   // 2 nlist: first tile and end of the used tiles of every list
    const uint32_t* pair_off;    // nlist + 1
    const uint32_t* item_off;    // nlist + 1: workgroups per list, prefix sums
    const uint32_t* sorted_pair; // pair index (q * nprobe + p) grouped by list
    uint32_t nlist, nprobe;
    uint32_t dummy_query;        // a padding row of the query table: zero operands, a threshold nothing meets
    const uint4* q8;             // [query][plane][granule]
    const uint32_t* tau;         // per query
    const float* ginv;           // 1 / (2 s2) of the batch (l2)
    uint32_t k;                  // capacity of a private list
    uint64_t* partial;           // [pair][chunk][lane / 32][k]: tile slots
    uint32_t* partial_cnt;       // [pair][chunk][lane / 32]
    uint32_t* gate;              // per query: raised when one of its lists overflowed; gate[dummy_query] counts them
};

template <int TEST, bool NIBBLE = false>
__global__ void __launch_bounds__(256, 2)
ivf_sq8_i8_kernel(IvfSq8Args p) {
    __shared__ I8Stage stage[2];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint32_t item = blockIdx.x;
    cu32_p ioff = as_const(p.item_off);
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
    uint32_t chunks = (list_end - list_begin + kIvfSq8ChunkTiles - 1) / kIvfSq8ChunkTiles;
    chunks = chunks < kIvfSq8Chunks ? chunks : kIvfSq8Chunks;
    const uint32_t per = chunks != 0 ? (list_end - list_begin + chunks - 1) / chunks : 0;
    const uint32_t chunk = chunks != 0 ? (item - ioff[b]) % chunks : 0;
    const uint32_t group = chunks != 0 ? (item - ioff[b]) / chunks : 0;
    uint32_t tile_begin = list_begin + chunk * per;
    tile_begin = tile_begin < list_end ? tile_begin : list_end;
    const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
    const uint32_t pbeg = as_const(p.pair_off)[b] + group * kIvfSq8Pairs + wave * kWave;
    const uint32_t pend = as_const(p.pair_off)[b + 1];
    const bool active = pbeg < pend;
    const uint32_t nstages = (tile_end - tile_begin + kI8StageTiles - 1) / kI8StageTiles;
    if (nstages == 0) {
        return;
    }
    constexpr bool kTerm = TEST == kI8TestIntTerm;

    intx4 qh[2][4], ql[2][4];
    uint32_t tau[2], qidx[2];
    uint32_t ncand[2] = {0, 0};
    uint64_t my_list[2];
    bool live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t idx = pbeg + 32 * j + l32;
        live[j] = idx < pend;
        const uint32_t pair = live[j] ? as_const(p.sorted_pair)[idx] : 0U;
        qidx[j] = live[j] ? pair / p.nprobe : p.dummy_query;
        const uint4* rowp = p.q8 + static_cast<uint64_t>(qidx[j]) * (kI8QueryBytes / 16);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint4 hv = rowp[2 * s + half];
            const uint4 lv = rowp[8 + 2 * s + half];
            qh[j][s] = intx4{static_cast<int>(hv.x), static_cast<int>(hv.y), static_cast<int>(hv.z),
                             static_cast<int>(hv.w)};
            ql[j][s] = intx4{static_cast<int>(lv.x), static_cast<int>(lv.y), static_cast<int>(lv.z),
                             static_cast<int>(lv.w)};
        }
        tau[j] = live[j] ? p.tau[qidx[j]] : 0x7FFFFFFFU;
        my_list[j] = (static_cast<uint64_t>(pair) * kIvfSq8Chunks + chunk) * 2 + half;
    }
    const float ginv = kTerm ? p.ginv[0] : 0.0F;

    uint4 regs[kI8StageTiles][2];
    float my_term[kI8StageTiles];
    auto fetch = [&](uint32_t sg) {
#pragma unroll
        for (int tt = 0; tt < kI8StageTiles; ++tt) {
            const uint32_t tile = tile_begin + sg * kI8StageTiles + tt;
            const bool real = tile < tile_end;
#pragma unroll
            for (int r = 0; r < (NIBBLE ? 1 : 2); ++r) {
                const uint32_t j = wave + 4 * r;
                const uint32_t none = NIBBLE ? 0U : 0x80808080U;
                regs[tt][r] = make_uint4(none, none, none, none);
                if (real && j < p.G) {
                    regs[tt][r] = p.tiles[(static_cast<uint64_t>(tile) * p.G + j) * kWave + lane];
                }
            }
            if constexpr (kTerm) {
                my_term[tt] = 0.0F;
                if (wave == 0) {
                    // Slots without a code hold zero codes: their term is that of the zero vector, and the rescoring
                    // leaves them out by their id.
                    my_term[tt] = real ? p.term[static_cast<uint64_t>(tile) * kWave + lane] : __builtin_inff();
                }
            }
        }
    };
    auto park = [&](I8Stage& st) {
#pragma unroll
        for (int tt = 0; tt < kI8StageTiles; ++tt) {
            if constexpr (NIBBLE) {
                // sq4: a granule is staged as two, its low and its high nibbles, as they are
                const uint4 v = regs[tt][0];
                const uint32_t m = 0x0F0F0F0FU;
                st.codes[tt][(2 * wave) * kWave + lane] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
                st.codes[tt][(2 * wave + 1) * kWave + lane] =
                    make_uint4((v.x >> 4) & m, (v.y >> 4) & m, (v.z >> 4) & m, (v.w >> 4) & m);
            } else {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const uint4 v = regs[tt][r];
                    st.codes[tt][(wave + 4 * r) * kWave + lane] =
                        make_uint4(v.x ^ 0x80808080U, v.y ^ 0x80808080U, v.z ^ 0x80808080U, v.w ^ 0x80808080U);
                }
            }
            if constexpr (kTerm) {
                if (wave == 0) {
                    const float x = my_term[tt] * ginv;
                    const int32_t io = x >= kI8TermClamp ? static_cast<int32_t>(kI8TermClamp) : __float2int_rn(x);
                    st.term[tt][lane] = __int_as_float(-io);
                }
            }
        }
    };

    constexpr int kBlocks = 4 * kI8StageTiles;
    fetch(0);
    park(stage[0]);
    __syncthreads();
    uint32_t cur = 0;
    for (uint32_t sg = 0; sg < nstages; ++sg) {
        if (sg + 1 < nstages) {
            fetch(sg + 1);
        }
        if (active) {
            const I8Stage& st = stage[cur];
            const uint64_t slot0 = (static_cast<uint64_t>(tile_begin) + sg * kI8StageTiles) * kWave;
            intx16 hi[2], lo[2];
            intx4 av[2][4];
            float tm[2][16];
            auto read_row = [&](int r) {
                const int tt = r >> 1, i = r & 1;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint4 c = st.codes[tt][(2 * s + half) * kWave + 32 * i + l32];
                    av[r & 1][s] = intx4{static_cast<int>(c.x), static_cast<int>(c.y), static_cast<int>(c.z),
                                         static_cast<int>(c.w)};
                }
                if constexpr (kTerm) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const float4 v = *reinterpret_cast<const float4*>(&st.term[tt][32 * i + 8 * g + 4 * half]);
                        tm[r & 1][4 * g] = v.x;
                        tm[r & 1][4 * g + 1] = v.y;
                        tm[r & 1][4 * g + 2] = v.z;
                        tm[r & 1][4 * g + 3] = v.w;
                    }
                }
            };
            auto multiply = [&](int blk, intx16& h, intx16& l) {
                const int r = blk >> 1, j = blk & 1;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    h[e] = 0;
                    l[e] = kTerm ? __float_as_int(tm[r & 1][e]) : 0;
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    h = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[r & 1][s], qh[j][s], h, 0, 0, 0);
                    l = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[r & 1][s], ql[j][s], l, 0, 0, 0);
                }
            };
            auto judged = [&](int blk, int e) { return (hi[blk & 1][e] << 8) + lo[blk & 1][e]; };
            read_row(0);
            multiply(0, hi[0], lo[0]);
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                const int r = blk >> 1, j = blk & 1;
                const bool reads = j == 0 && blk + 2 < kBlocks;
                if (reads) {
                    read_row(r + 1);
                }
                if (blk + 1 < kBlocks) {
                    multiply(blk + 1, hi[(blk + 1) & 1], lo[(blk + 1) & 1]);
                }
                int32_t gbest[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    gbest[g] = max(max(max(judged(blk, 4 * g), judged(blk, 4 * g + 1)), judged(blk, 4 * g + 2)),
                                   judged(blk, 4 * g + 3));
                }
                const bool hit = max(max(max(gbest[0], gbest[1]), gbest[2]), gbest[3]) >= static_cast<int32_t>(tau[j]);
                const uint64_t any = __ballot(hit);
                if (blk + 1 < kBlocks) {
                    if (reads) {
                        __builtin_amdgcn_sched_group_barrier(0x100, kTerm ? 8 : 4, 0);
                    }
#pragma unroll
                    for (int m = 0; m < 8; ++m) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                    }
                }
                if (any != 0) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        if (__ballot(gbest[g] >= static_cast<int32_t>(tau[j])) == 0) {
                            continue;
                        }
#pragma unroll
                        for (int e = 4 * g; e < 4 * g + 4; ++e) {
                            const bool pass = judged(blk, e) >= static_cast<int32_t>(tau[j]) && live[j];
                            if (__ballot(pass) != 0 && pass) {
                                const uint64_t slot = slot0 + 32 * r + 8 * (e >> 2) + 4 * half + (e & 3);
                                // The second tile of the last stage may lie behind the chunk: its staged codes and term
                                // fail every threshold but that of a query without a bound, which everything passes --
                                // and behind the chunk lies the next chunk, or the next list.
                                if (slot >= static_cast<uint64_t>(tile_end) * kWave) {
                                    continue;
                                }
                                if (ncand[j] < p.k) {
                                    p.partial[my_list[j] * p.k + ncand[j]] = slot;
                                }
                                ++ncand[j];
                            }
                        }
                    }
                }
            }
        }
        if (sg + 1 < nstages) {
            park(stage[cur ^ 1]);
        }
        __syncthreads();
        cur ^= 1;
    }
    if (active) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (live[j]) {
                // k + 1 for a list that overflowed: that is how the pair is told from the query's other pairs afterwards
                p.partial_cnt[my_list[j]] = ncand[j] <= p.k ? ncand[j] : p.k + 1;
                if (ncand[j] > p.k) {
                    if (atomicExch(&p.gate[qidx[j]], 1U) == 0U) {
                        atomicAdd(&p.gate[p.dummy_query], 1U);
                    }
                }
            }
        }
    }
}

bool
ivf_sq8_i8_supports(const vsag_amd_store* s) {
    const bool kind_ok = (s->kind == VSAG_AMD_KIND_SQ8 && s->G <= 8) || (s->kind == VSAG_AMD_KIND_SQ4 && s->G <= 4);
    return kind_ok && s->nlist > 0 && s->dpad <= kI8Dims && s->pf_term != nullptr && s->pf_ymax != nullptr &&
           s->residual_centroids_dev == nullptr;
}

// Bytes of the query planes, floats of the scalars and words of the thresholds for nq queries and one padding row.
size_t
ivf_sq8_i8_query_bytes(uint64_t nq) {
    return prefilter_i8_query_bytes(nq + 1);
}

size_t
ivf_sq8_i8_scalar_floats(uint64_t nq) {
    return prefilter_i8_scalar_floats(nq + 1);
}

size_t
ivf_sq8_i8_tau_words(uint64_t nq) {
    return static_cast<size_t>(div_up(nq + 1, static_cast<uint64_t>(kI8Group)) * kI8Group);
}

// Quantizes the queries against their bounds (one scale for the batch) and collects, for the pairs of probe columns
// [p0, nprobe) grouped by list (pair_off, sorted_pair; item_off as for ivf_i8.hip), the tile slots whose distance may
// still matter: private list (pair * 8 + chunk * 2 + lane / 32) of kcand records in `partial`, counts in partial_cnt
// (zero before).  gate: nq + 2 words as in ivf_i8.hip.
int
launch_ivf_sq8_i8(const vsag_amd_store* s, const float* qtab, uint32_t qstride, const float* qmeta, uint32_t qmeta_stride,
                  uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off, const uint32_t* item_off,
                  const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, uint8_t* q8, float* u, uint32_t* tau,
                  uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t nq_pad = ivf_sq8_i8_tau_words(nq);
    float* ginv = u + nq_pad;
    const uint64_t head = (nq_pad + nq_pad / kI8Group + 1) / 2 * 2;
    QuantizeArgs z{};
    z.qtab = qtab;
    z.qstride = qstride;
    z.kdim = s->dpad;
    z.scale = l2 ? s->scale_dev : nullptr;
    z.qmeta = l2 ? nullptr : qmeta;
    z.qmeta_stride = qmeta_stride;
    z.is_l2 = l2 ? 1 : 0;
    z.nibbles = s->kind == VSAG_AMD_KIND_SQ4 ? 1 : 0;
    z.bound = bound;
    z.ymax_bits = s->pf_ymax;
    z.nq = nq;
    z.nq_pad = nq_pad;
    z.q8 = q8;
    z.amax = u;
    z.ginv = ginv;
    z.tau = tau;
    z.scal = reinterpret_cast<double*>(u + head);
    if (l2) {
        hipLaunchKernelGGL(query_amax_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(kWave), 0, st, z);
        hipLaunchKernelGGL(spread_amax_kernel, dim3(1), dim3(1024), 0, st, u, nq_pad);
    }
    hipLaunchKernelGGL(quantize_queries_i8_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(kWave), 0, st, z);
    VA_HIP(hipGetLastError());
    IvfSq8Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.term = s->pf_term;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.dummy_query = static_cast<uint32_t>(nq);
    p.q8 = reinterpret_cast<const uint4*>(q8);
    p.tau = tau;
    p.ginv = ginv;
    p.k = kcand;
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kIvfSq8Pairs)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfSq8Chunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    if (z.nibbles) {
        if (l2) {
            hipLaunchKernelGGL((ivf_sq8_i8_kernel<kI8TestIntTerm, true>), grid, dim3(256), 0, st, p);
        } else {
            hipLaunchKernelGGL((ivf_sq8_i8_kernel<kI8TestInt, true>), grid, dim3(256), 0, st, p);
        }
    } else if (l2) {
        hipLaunchKernelGGL(ivf_sq8_i8_kernel<kI8TestIntTerm>, grid, dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL(ivf_sq8_i8_kernel<kI8TestInt>, grid, dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

// Bytes of the quantized query table for nq queries.
size_t
prefilter_i8_query_bytes(uint64_t nq) {
    return static_cast<size_t>(div_up(nq, static_cast<uint64_t>(kI8Group)) * kI8Group) * kI8QueryBytes;
}

// Floats of per-query and per-group scalars the quantizing kernels keep for nq queries.
size_t
prefilter_i8_scalar_floats(uint64_t nq) {
    const uint64_t groups = div_up(nq, static_cast<uint64_t>(kI8Group));
    // a float per padded query, one per group, then (8-byte aligned) kI8Scalars doubles per padded query
    const uint64_t head = (groups * kI8Group + groups + 1) / 2 * 2;
    return static_cast<size_t>(head + 2 * kI8Scalars * groups * kI8Group);
}

// Candidate lists per query (two per workgroup column) for nq queries over `span` tiles.
uint32_t
prefilter_i8_sub_lists(uint64_t nq, uint64_t span) {
    const uint64_t qgroups = div_up(nq, static_cast<uint64_t>(kI8Group));
    // Two workgroups fit a compute unit.  The workgroups of a launch take about equally long, so they run in rounds of
    // 2 x compute units: the number of columns is the multiple of eight (whole turns of the XCDs, see the kernel's
    // workgroup mapping) between six and twelve rounds that leaves the last round fullest (few rounds: the slowest
    // workgroup of the last one is a larger share of the launch; many: every workgroup loads its queries anew).
    constexpr uint64_t rounds_lo = 6, rounds_hi = 12;
    const uint64_t per_round = static_cast<uint64_t>(device_cu_count()) * 2;
    const uint64_t stages = div_up(span, static_cast<uint64_t>(kI8StageTiles));
    uint64_t groups = std::max<uint64_t>(1, std::min<uint64_t>(per_round * rounds_lo / qgroups, stages));
    // A workgroup loads the planes of its 256 queries (64 KB) before its first stage, and every column is two more
    // private lists per query whose counts the rescoring reads: on a short level a workgroup walks at least sixteen
    // stages, as long as two rounds of workgroups remain (1M codes, 10 000 queries: 2.89 -> 2.84 ms per call).
    const uint64_t by_length = std::max<uint64_t>(1, stages / 16);
    if (groups > by_length) {
        groups = std::max(by_length, std::min(groups, div_up(per_round * 2, qgroups)));
    }
    if (groups >= 8) {
        uint64_t best = groups / 8 * 8;
        double best_fill = 0.0;
        for (uint64_t g = best; g <= stages && g * qgroups <= per_round * rounds_hi; g += 8) {
            const uint64_t rem = g * qgroups % per_round;
            const double fill = rem == 0 ? 1.0 : static_cast<double>(rem) / static_cast<double>(per_round);
            if (fill > best_fill + 1e-9) {
                best_fill = fill;
                best = g;
            }
        }
        groups = best;
    }
    return static_cast<uint32_t>(2 * groups);
}

// Quantizes the queries against their current bounds and collects the candidates of tiles [tile_begin, tile_end)
// into sub_lists lists of sub_cap slots per query (sub_lists as prefilter_i8_sub_lists gives it).  first_level: the
// first level of a call quantizes; the later ones keep the planes and only redo the thresholds, after lowering the
// bounds to the k-th of merged_dists (k per query; null: the bounds are up to date).
int
launch_prefilter_i8(const vsag_amd_store* s, const float* qtab, uint32_t qstride, const float* qmeta,
                    uint32_t qmeta_stride, uint64_t nq, uint64_t tile_begin, uint64_t tile_end, const uint32_t* bound,
                    uint8_t* q8, float* u, uint32_t* tau, uint32_t* cand, uint32_t* cand_cnt, uint32_t sub_lists,
                    uint32_t sub_cap, bool first_level, const float* merged_dists, uint32_t k, uint32_t* bound_rw,
                    hipStream_t st) {
    const bool nibbles = s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4;
    const bool uniform = s->kind == VSAG_AMD_KIND_SQ8_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4_UNIFORM;
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t nq_pad = div_up(nq, static_cast<uint64_t>(kI8Group)) * kI8Group;
    // `u` holds a float per padded query and one per group of kI8Group queries behind them (prefilter_i8_scalar_floats).
    float* ginv = u + nq_pad;
    const uint64_t head = (nq_pad + nq_pad / kI8Group + 1) / 2 * 2;
    double* scal = reinterpret_cast<double*>(u + head);
    const dim3 per_query(static_cast<uint32_t>(div_up(nq, 256)));
    if (uniform) {
        UniformQuantizeArgs z{};
        z.qtab = reinterpret_cast<const uint32_t*>(qtab);
        z.qstride = qstride;
        z.kdim = s->dpad;
        z.qmeta = qmeta;
        z.qmeta_stride = qmeta_stride;
        z.is_l2 = l2 ? 1 : 0;
        z.nibbles = nibbles ? 1 : 0;
        z.lb = s->ulb;
        z.rate = s->scalar_rate;
        z.lb2 = s->ulb * s->ulb;
        z.bound = bound;
        z.nq = nq;
        z.nq_pad = nq_pad;
        z.q8 = q8;
        z.u = u;
        z.tau = tau;
        z.scal = scal;
        if (first_level) {
            hipLaunchKernelGGL(quantize_uniform_i8_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(kWave), 0, st, z);
        } else {
            hipLaunchKernelGGL(retau_uniform_i8_kernel, per_query, dim3(256), 0, st, z, merged_dists, k, bound_rw);
        }
    } else {
        QuantizeArgs z{};
        z.qtab = qtab;
        z.qstride = qstride;
        z.kdim = s->dpad;
        z.scale = l2 ? s->scale_dev : nullptr;
        z.qmeta = l2 ? nullptr : qmeta;
        z.qmeta_stride = qmeta_stride;
        z.is_l2 = l2 ? 1 : 0;
        z.nibbles = nibbles ? 1 : 0;
        z.bound = bound;
        z.ymax_bits = s->pf_ymax;
        z.nq = nq;
        z.nq_pad = nq_pad;
        z.q8 = q8;
        z.amax = u;
        z.ginv = ginv;
        z.tau = tau;
        z.scal = scal;
        if (first_level) {
            if (l2) {
                hipLaunchKernelGGL(query_amax_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(kWave), 0, st, z);
            }
            hipLaunchKernelGGL(quantize_queries_i8_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(kWave), 0, st, z);
        } else {
            hipLaunchKernelGGL(retau_queries_i8_kernel, per_query, dim3(256), 0, st, z, merged_dists, k, bound_rw);
        }
    }
    VA_HIP(hipGetLastError());

    PrefilterI8Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.tile_begin = tile_begin;
    p.tile_end = tile_end;
    p.n = s->n;
    p.q8 = reinterpret_cast<const uint4*>(q8);
    p.nq = nq;
    p.term = s->pf_term;
    p.u = u;
    p.ginv = ginv;
    p.tau = tau;
    p.cand = cand;
    p.cand_cnt = cand_cnt;
    p.sub_cap = sub_cap;
    p.groups = sub_lists / 2;
    VA_CHECK_ARG(sub_lists == prefilter_i8_sub_lists(nq, tile_end - tile_begin), "candidate lists do not match the grid");
    p.qgroups = static_cast<uint32_t>(nq_pad / kI8Group);
    dim3 grid(p.groups * p.qgroups);
    timing_begin(st);
    if (nibbles && uniform) {
        hipLaunchKernelGGL((prefilter_i8_kernel<kI8TestFma, true>), grid, dim3(256), 0, st, p);
    } else if (nibbles && l2) {
        hipLaunchKernelGGL((prefilter_i8_kernel<kI8TestIntTerm, true>), grid, dim3(256), 0, st, p);
    } else if (nibbles) {
        hipLaunchKernelGGL((prefilter_i8_kernel<kI8TestInt, true>), grid, dim3(256), 0, st, p);
    } else if (uniform) {
        hipLaunchKernelGGL(prefilter_i8_kernel<kI8TestFma>, grid, dim3(256), 0, st, p);
    } else if (l2) {
        hipLaunchKernelGGL(prefilter_i8_kernel<kI8TestIntTerm>, grid, dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL(prefilter_i8_kernel<kI8TestInt>, grid, dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
