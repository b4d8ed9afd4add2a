// CPU restatement of the VSAG search-core arithmetic (k-means assignment, FP32 / SQ8 / SQ4 /
// SQ4-uniform / SQ8-uniform / RaBitQ distance computers, bounded-heap top-k, IVF route/scan/rerank).
//
// THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP library is compared with, and the
// CPU baseline that bench.py times beside the GPU.  Nothing in the product path links, loads or
// calls it; the shipped library fails loudly when its HIP code object is missing instead of coming
// here.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it.
//
// Every function cites the reference file:line (relative to the VSAG source tree) whose arithmetic
// it restates.  How each one is pinned (known answers of the reference's own tests, the compiled
// reference scalar kernels, closed forms, brute force) is listed beside the tests that do it:
//   pinned by reference known answers ... sq_encode (NaN->0, 0.5->127/7), squ_encode byte images,
//                                          rabitq 4-bit query planes, rabitq_binary_ip 0/36/32
//   pinned by compiled reference kernels . fp32/sq8/sq4 distances, sq4u/sq8u code IP, binary IPs,
//                                          normalize-with-centroid
//   pinned by closed form / brute force .. sq_train (sorted order statistics), kmeans_assign and its
//                                          loss (fp64 argmin and mean of the minima), heaps (sort), ivf
//                                          composition (nprobe=nlist), rabitq_dist (a stored vector as
//                                          32-bit query: estimate exactly 0 / 1 - |x|^2; the +-1 clamp of
//                                          a tiny error field; zero raw norms -> 1; the 4-bit branch
//                                          against the fp32 branch on the dequantised query),
//                                          kmeans_init_pp (numpy restatement with cumsum / searchsorted in
//                                          float64; k = n picks every row once; coincident rows)
//   pqfs ................................. pqfs_lookup32 against the reference's compiled PQFastScanLookUp32 and
//                                          committed vectors; Package32 / Unpack32 by round trip and the mapper
//                                          order; encode, query table and distance by brute-force argmin and the
//                                          closed form (table entry = the exact subspace distance within one
//                                          quantisation step); the reference test's own error bound
//   multi-bit rabitq ..................... the float x plane / float x code inner products against the reference's
//                                          compiled RaBitQFloatSplitCodeIP / RaBitQFloatSQIP; the fast encoder on
//                                          the known input of the reference's test; both encoders against the
//                                          exhaustive optimum on tiny inputs (the extended one against hand-traced
//                                          answers of the reference's walk, which is not optimal); zero vectors;
//                                          the estimator's closed form (ip_obar_q) and a stored vector's self
//                                          distance
//   rabitq decode (residual lists) ....... the scale step against the reference's compiled
//                                          InverseNormalizeWithCentroid; the whole against what the definition
//                                          fixes: R x - centroid has the code's signs and one magnitude, norm / sqrt(d),
//                                          and a row built to sit exactly on such a point decodes to itself
//   FhtKacRotator (rabitq_use_fht) ....... the four primitives against the reference's compiled FlipSign, VecRescale,
//                                          FHTRotate and KacsWalk; the transform by the reference test's own
//                                          properties (lengths kept, the inverse returns the input within 1e-4) and
//                                          the closed form without flips on a power of two ((H / sqrt(d))^4 = I)
//   parity unpinned ...................... nothing; what the formulas leave open is the order of fp32
//                                          operations inside rabitq_dist and the k-means loss (no
//                                          executable reference class), which the 1e-4 relative
//                                          tolerance of the comparisons covers
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <queue>
#include <random>
#include <utility>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

enum Metric { kL2 = 0, kIP = 1, kCosine = 2 };

inline uint64_t
align_up(uint64_t v, uint64_t a) {
    return (v + a - 1) / a * a;
}

// ---------------------------------------------------------------- FP32 primitives
// src/simd/generic.cpp:99-107 with the Width=1 traits (src/simd/traits/simd_traits_generic.h:42-96):
// one running fp32 sum, sub then multiply-add per element, element order 0..dim-1.
inline float
fp32_l2sqr(const float* q, const float* x, uint64_t dim) {
    float s = 0.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        float t = q[i] - x[i];
        s = t * t + s;
    }
    return s;
}

inline float
fp32_ip(const float* q, const float* x, uint64_t dim) {
    float s = 0.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        s = q[i] * x[i] + s;
    }
    return s;
}

// src/simd/generic.cpp:874-878: norm = sqrt(<x,x>), to = from / norm (a zero norm divides by 1).
inline float
normalize(const float* from, float* to, uint64_t dim) {
    float norm = std::sqrt(fp32_ip(from, from, dim));
    float scalar = norm == 0 ? 1.0F : norm;  // DivScalarImpl, src/simd/kernels/scalar_op.h:40-42
    for (uint64_t i = 0; i < dim; ++i) {
        to[i] = from[i] / scalar;
    }
    return norm;
}

// src/simd/kernels/normalize.h:35-83: norm of (from - centroid); norm_sq < 1e-5 -> norm = 1.
inline float
normalize_with_centroid(const float* from, const float* centroid, float* to, uint64_t dim) {
    float norm_sq = 0.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        float d = from[i] - centroid[i];
        norm_sq = d * d + norm_sq;
    }
    float norm = (norm_sq < 1e-5F) ? 1.0F : std::sqrt(norm_sq);
    for (uint64_t i = 0; i < dim; ++i) {
        to[i] = (from[i] - centroid[i]) / norm;
    }
    return norm;
}

// ---------------------------------------------------------------- scalar quantization
// src/quantization/scalar_quantization/scalar_quantization_utils.h:19-30
inline float
clamp_delta(float delta) {
    if (!(delta >= 0.0F)) {
        return 0.0F;
    }
    if (delta > 0.999F) {
        return 1.0F;
    }
    return delta;
}

// src/simd/kernels/sq8_compute.h:44-137 (Width=1): code/255 then *diff+lb, fp32.
inline float
sq8_ip(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    float s = 0.0F;
    const float inv255 = 1.0F / 255.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        float normalized = static_cast<float>(c[i]) * inv255;
        float adjusted = normalized * diff[i] + lb[i];
        s = q[i] * adjusted + s;
    }
    return s;
}

inline float
sq8_l2sqr(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    float s = 0.0F;
    const float inv255 = 1.0F / 255.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        float normalized = static_cast<float>(c[i]) * inv255;
        float adjusted = normalized * diff[i] + lb[i];
        float d = q[i] - adjusted;
        s = d * d + s;
    }
    return s;
}

// src/simd/generic.cpp:316-340 (scalar SQ4): nibble * (1/15) * diff + lb, low nibble = even dim.
inline float
sq4_value(const uint8_t* c, const float* lb, const float* diff, uint64_t i) {
    uint8_t nibble = (i & 1) ? (c[i >> 1] >> 4) : (c[i >> 1] & 0x0f);
    return nibble * (1.0F / 15.0F) * diff[i] + lb[i];
}

inline float
sq4_ip(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    float s = 0.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        s += q[i] * sq4_value(c, lb, diff, i);
    }
    return s;
}

inline float
sq4_l2sqr(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    float s = 0.0F;
    for (uint64_t i = 0; i < dim; ++i) {
        float d = q[i] - sq4_value(c, lb, diff, i);
        s += d * d;
    }
    return s;
}

// src/simd/generic.cpp:406-431: integer code x code inner products.
inline int32_t
sq4u_codes_ip(const uint8_t* a, const uint8_t* b, uint64_t dim) {
    int32_t r = 0;
    for (uint64_t d = 0; d < dim; d += 2) {
        int32_t x_lo = a[d >> 1] & 0x0f;
        int32_t x_hi = (a[d >> 1] & 0xf0) >> 4;
        int32_t y_lo = b[d >> 1] & 0x0f;
        int32_t y_hi = (b[d >> 1] & 0xf0) >> 4;
        r += x_lo * y_lo + x_hi * y_hi;
    }
    return r;
}

inline int32_t
sq8u_codes_ip(const uint8_t* a, const uint8_t* b, uint64_t dim) {
    int32_t r = 0;
    for (uint64_t d = 0; d < dim; ++d) {
        r += static_cast<int32_t>(a[d]) * static_cast<int32_t>(b[d]);
    }
    return r;
}

// Byte layout of the uniform codes.
// sq4_uniform_quantizer.cpp:33-72 ; sq8_uniform_quantizer.cpp:30-62.
struct UniformLayout {
    uint64_t code_bytes;        // bytes holding nibbles / bytes (before alignment)
    uint64_t offset_norm;       // u64 sum code^2 (L2; SQ4U also for cosine)
    uint64_t offset_sum;        // f32 sum of raw values (IP / cosine)
    uint64_t offset_codes_sum;  // f32 sum of codes (SQ4U IP / cosine only)
    uint64_t code_size;
    bool has_norm, has_sum, has_codes_sum;
};

inline UniformLayout
uniform_layout(uint64_t dim, int bits, int metric) {
    UniformLayout l{};
    uint64_t align = 1;
    bool norm = (metric == kL2) || (bits == 4 && metric == kCosine);
    bool sum = (metric == kIP || metric == kCosine);
    if (norm) {
        align = std::max<uint64_t>(align, 8);
    }
    if (sum) {
        align = std::max<uint64_t>(align, 4);
    }
    l.code_bytes = (bits == 4) ? (dim + 1) / 2 : dim;
    l.code_size = align_up(l.code_bytes, align);
    l.has_norm = norm;
    l.has_sum = sum;
    l.has_codes_sum = sum && bits == 4;
    if (norm) {
        l.offset_norm = l.code_size;
        l.code_size += align_up(8, align);
    }
    if (sum) {
        l.offset_sum = l.code_size;
        l.code_size += align_up(4, align);
        if (bits == 4) {
            l.offset_codes_sum = l.code_size;
            l.code_size += align_up(4, align);
        }
    }
    return l;
}

// ---------------------------------------------------------------- RaBitQ
// rabitq_quantizer.cpp:102-176: field offsets of the base code and of the processed query ("standard" version: no
// PCA, no MRQ term, no split storage).  Every function below that takes `query_bits` reads the bits per dimension
// of the base code from its second byte: query_bits = 4 or 32, plus 256 * base_bits (0 stands for 1 bit).
struct RabitqLayout {
    uint64_t dim;
    int base_bits;
    uint64_t offset_norm_code;  // base_bits != 1 only
    uint64_t offset_norm, offset_error, offset_sum, offset_raw_norm, code_size;
    bool has_sum, has_raw_norm;
    uint64_t aligned_dim, plane_bytes;
    uint64_t q_offset_lb, q_offset_delta, q_offset_sum, q_offset_norm, q_offset_raw_norm, query_code_size;
};

inline RabitqLayout
rabitq_layout(uint64_t dim, int metric, int query_bits) {
    RabitqLayout l{};
    l.dim = dim;
    l.base_bits = (query_bits >> 8) == 0 ? 1 : (query_bits >> 8);
    query_bits &= 255;
    const uint64_t a = 4;
    uint64_t cs = align_up((dim + 7) / 8 * l.base_bits, a);
    if (l.base_bits != 1) {
        l.offset_norm_code = cs;
        cs += 4;
    }
    l.offset_norm = cs;
    cs += 4;
    l.offset_error = cs;
    cs += 4;
    l.has_sum = query_bits != 32;
    if (l.has_sum) {
        l.offset_sum = cs;
        cs += 4;
    }
    l.has_raw_norm = (metric == kIP || metric == kCosine);
    if (l.has_raw_norm) {
        l.offset_raw_norm = cs;
        cs += 4;
    }
    l.code_size = cs;
    uint64_t qs = 0;
    if (query_bits == 4) {
        l.aligned_dim = (dim + 511) / 512 * 512;
        l.plane_bytes = l.aligned_dim / 8;
        qs = l.aligned_dim / 8 * 4;
        l.q_offset_lb = qs;
        qs += 4;
        l.q_offset_delta = qs;
        qs += 4;
        l.q_offset_sum = qs;
        qs += 4;
    } else {
        qs = align_up(4 * dim, a);
        if (l.base_bits != 1) {
            l.q_offset_sum = qs;
            qs += 4;
        }
    }
    l.q_offset_norm = qs;
    qs += 4;
    if (l.has_raw_norm) {
        l.q_offset_raw_norm = qs;
        qs += 4;
    }
    l.query_code_size = qs;
    return l;
}

// src/simd/generic.cpp:447-471
inline float
rabitq_float_binary_ip(const float* v, const uint8_t* bits, uint64_t dim, float inv_sqrt_d) {
    if (dim == 0) {
        return 0.0F;
    }
    float pos, neg;
    if (inv_sqrt_d > 1e-3) {
        pos = inv_sqrt_d;
        neg = -inv_sqrt_d;
    } else {
        pos = 1.0F;
        neg = 0;
    }
    float r = 0.0F;
    for (uint64_t d = 0; d < dim; ++d) {
        bool bit = ((bits[d / 8] >> (d % 8)) & 1) != 0;
        r += (bit ? pos : neg) * v[d];
    }
    return r;
}

// src/simd/generic.cpp:832-872: sum_b popcount(plane_b & bits) << b; planes are ceil(dim/8) bytes apart.
inline uint32_t
rabitq_sq4u_binary_ip(const uint8_t* planes, const uint8_t* bits, uint64_t dim) {
    if (dim == 0) {
        return 0;
    }
    uint64_t num_bytes = (dim + 7) / 8;
    uint32_t r = 0;
    for (uint64_t b = 0; b < 4; ++b) {
        uint32_t cnt = 0;
        for (uint64_t i = 0; i < num_bytes; ++i) {
            cnt += __builtin_popcount(static_cast<unsigned>(planes[b * num_bytes + i] & bits[i]));
        }
        r += cnt << b;
    }
    return r;
}

// src/simd/generic.cpp:799-811
inline float
rabitq_float_sq_ip(const float* v, const uint8_t* codes, uint64_t dim) {
    float r = 0.0F;
    for (uint64_t d = 0; d < dim; ++d) {
        r += static_cast<float>(codes[d]) * v[d];
    }
    return r;
}

// src/simd/generic.cpp:743-771 as RaBitQFloatSQIPByPlanes calls it without split storage (rabitq_quantizer.cpp:354-374):
// plane b of ceil(dim / 8) bytes holds bit b of every dimension's code (PackIntoPlanes, :431-453); the top plane is
// the "one bit" code, the planes below it the supplement.
inline float
rabitq_float_planes_ip(const float* v, const uint8_t* planes, uint64_t dim, int base_bits) {
    if (dim == 0) {
        return 0.0F;
    }
    const uint64_t plane_bytes = (dim + 7) / 8;
    const uint32_t supplement_bits = static_cast<uint32_t>(base_bits - 1);
    const uint8_t* one_bit = planes + supplement_bits * plane_bytes;
    float r = 0.0F;
    for (uint64_t d = 0; d < dim; ++d) {
        const uint64_t byte = d >> 3;
        const uint8_t mask = static_cast<uint8_t>(1U << (d & 7));
        uint32_t code = (one_bit[byte] & mask) != 0 ? 1U << supplement_bits : 0U;
        for (uint32_t bit = 0; bit < supplement_bits; ++bit) {
            if ((planes[bit * plane_bytes + byte] & mask) != 0) {
                code += 1U << bit;
            }
        }
        r += v[d] * static_cast<float>(code);
    }
    return r;
}

// rabitq_quantizer.cpp:256-267
inline float
ip_obar_q(float ip_yu_q, float q_prime_sum, float y_norm, int bits) {
    const float c = 0.5F * static_cast<float>((1U << bits) - 1U);
    if (y_norm <= 0.0F) {
        return 0.0F;
    }
    float ret = ip_yu_q - c * q_prime_sum;
    ret /= y_norm;
    return ret;
}

// RaBitQuantizer::FastEncodeRaBitQ (rabitq_quantizer.cpp:609-704): a floor grid over [-max|o|, max|o|], then rounds of
// one-level moves per coordinate that raise <o, y>^2 / |y|^2 (y = code - centre), all sums in double.
inline void
rabitq_fast_encode(const float* o, uint64_t dim, int bits, uint64_t rounds, uint8_t* code, float* y_norm) {
    constexpr double adjustment_epsilon = 1e-8;
    const uint32_t code_max = (1U << bits) - 1U;
    const double center = 0.5 * static_cast<double>(code_max);
    double max_abs = 0.0;
    for (uint64_t d = 0; d < dim; ++d) {
        max_abs = std::max(max_abs, std::fabs(static_cast<double>(o[d])));
    }
    if (max_abs <= 0.0) {
        for (uint64_t d = 0; d < dim; ++d) {
            code[d] = static_cast<uint8_t>(code_max / 2U);
        }
        *y_norm = 1.0F;
        return;
    }
    const double delta = 2.0 * max_abs / static_cast<double>(code_max + 1U);
    const double inv_delta = 1.0 / delta;
    double ip = 0.0, norm_sqr = 0.0;
    for (uint64_t d = 0; d < dim; ++d) {
        const double scaled = (static_cast<double>(o[d]) + max_abs) * inv_delta;
        int64_t q = static_cast<int64_t>(std::floor(scaled));
        q = std::min<int64_t>(std::max<int64_t>(q, 0), code_max);
        code[d] = static_cast<uint8_t>(q);
        const double centered = static_cast<double>(q) - center;
        ip += static_cast<double>(o[d]) * centered;
        norm_sqr += centered * centered;
    }
    auto score = [](double inner, double squared) { return squared > 0.0 ? inner * inner / squared : 0.0; };
    for (uint64_t round = 0; round < rounds; ++round) {
        bool adjusted = false;
        for (uint64_t d = 0; d < dim; ++d) {
            const int32_t cur = code[d];
            const double cur_value = static_cast<double>(cur) - center;
            int32_t best_code = cur;
            double best_ip = ip, best_norm = norm_sqr, best_score = score(ip, norm_sqr);
            for (int32_t dir = -1; dir <= 1; dir += 2) {
                const int32_t cand = cur + dir;
                if (cand < 0 || cand > static_cast<int32_t>(code_max)) {
                    continue;
                }
                const double cand_ip = ip + static_cast<double>(dir) * static_cast<double>(o[d]);
                if (cand_ip < 0.0) {
                    continue;
                }
                const double cand_norm = norm_sqr + 2.0 * cur_value * static_cast<double>(dir) + 1.0;
                const double cand_score = score(cand_ip, cand_norm);
                const double tolerance = adjustment_epsilon * std::max(1.0, std::fabs(best_score));
                if (cand_score > best_score + tolerance) {
                    best_code = cand;
                    best_ip = cand_ip;
                    best_norm = cand_norm;
                    best_score = cand_score;
                }
            }
            if (best_code != cur) {
                code[d] = static_cast<uint8_t>(best_code);
                ip = best_ip;
                norm_sqr = best_norm;
                adjusted = true;
            }
        }
        if (!adjusted) {
            break;
        }
    }
    norm_sqr = 0.0;
    for (uint64_t d = 0; d < dim; ++d) {
        const double centered = static_cast<double>(code[d]) - center;
        norm_sqr += centered * centered;
    }
    *y_norm = static_cast<float>(std::sqrt(norm_sqr));
    if (!std::isfinite(*y_norm) || *y_norm <= 0.0F) {
        *y_norm = 1.0F;
    }
}

// RaBitQuantizer::EncodeExtendRaBitQ (rabitq_quantizer.cpp:455-607): walks the scale t upwards, one grid step of one
// coordinate per event (events ordered by (t, coordinate)), keeps the t with the largest <y2, o> / |y2|, then rounds
// 2 t o to the grid of the parity of 2^bits - 1.
inline void
rabitq_extend_encode(const float* o, uint64_t dim, int bits, uint8_t* code, float* y_norm) {
    constexpr double eps = 1e-12;
    const int y2_max = static_cast<int>((1U << bits) - 1U);
    const double c = 0.5 * static_cast<double>(y2_max);
    const int step = 2;
    auto clamp_int = [](int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); };
    auto round_clamp_parity = [&](double val) {
        const int lo = -y2_max, hi = +y2_max;
        const long long r = std::llround(val);
        const int ri = clamp_int(static_cast<int>(r), lo, hi);
        if ((ri & 1) == (y2_max & 1)) {
            return ri;
        }
        const int s = (val >= 0.0) ? +1 : -1;
        int cand = ri + s;
        if (cand < lo || cand > hi) {
            cand = ri - s;
        }
        return clamp_int(cand, lo, hi);
    };
    double max_o = 0.0;
    for (uint64_t i = 0; i < dim; ++i) {
        max_o = std::max(max_o, std::fabs(static_cast<double>(o[i])));
    }
    if (max_o <= 0.0) {
        for (uint64_t i = 0; i < dim; ++i) {
            code[i] = static_cast<uint8_t>(y2_max / 2);
        }
        *y_norm = 1.0F;
        return;
    }
    std::vector<int> y2_cur(dim, 0);
    const double t_end = (static_cast<double>(y2_max) + 2.0) / (2.0 * max_o);
    double ip_y2_o = 0.0, norm_y2 = 0.0;
    typedef std::pair<double, size_t> Event;
    std::priority_queue<Event, std::vector<Event>, std::greater<Event>> pq;
    auto next_t = [&](size_t i) {
        const double oi = static_cast<double>(o[i]);
        if (std::fabs(oi) < 1e-3) {
            return std::numeric_limits<double>::infinity();
        }
        const int sign = (oi > 0.0) ? +1 : -1;
        const int y2_next = y2_cur[i] + sign * step;
        if (y2_next < -y2_max || y2_next > +y2_max) {
            return std::numeric_limits<double>::infinity();
        }
        double t = static_cast<double>(y2_cur[i] + sign) / (2.0 * oi);
        if (t < 0.0) {
            t = 0.0;
        }
        return t;
    };
    for (size_t i = 0; i < dim; ++i) {
        if (static_cast<double>(o[i]) == 0.0) {
            continue;
        }
        const double t0 = next_t(i);
        if (std::isfinite(t0) && t0 <= t_end) {
            pq.emplace(t0, i);
        }
    }
    double best_ip = eps, best_t = 0.0;
    while (!pq.empty()) {
        const double cur_t = pq.top().first;
        const size_t k = pq.top().second;
        pq.pop();
        if (cur_t >= t_end) {
            break;
        }
        const int sign = (o[k] > 0.0) ? +1 : -1;
        const int y2_old = y2_cur[k];
        const int y2_new = y2_old + sign * step;
        if (y2_new < -y2_max || y2_new > +y2_max) {
            continue;
        }
        y2_cur[k] = y2_new;
        ip_y2_o += (static_cast<double>(y2_new) - static_cast<double>(y2_old)) * o[k];
        norm_y2 += static_cast<double>(y2_new) * static_cast<double>(y2_new) -
                   static_cast<double>(y2_old) * static_cast<double>(y2_old);
        const double cur_ip = (norm_y2 > 0.0) ? (ip_y2_o / std::sqrt(norm_y2)) : 0.0;
        if (cur_ip > best_ip) {
            best_ip = cur_ip;
            best_t = cur_t;
        }
        double t_next = next_t(k);
        if (t_next <= cur_t) {
            t_next = std::nextafter(cur_t, std::numeric_limits<double>::infinity());
        }
        if (std::isfinite(t_next) && t_next < t_end) {
            pq.emplace(t_next, k);
        }
    }
    for (size_t i = 0; i < dim; ++i) {
        const double val = 2.0 * best_t * static_cast<double>(o[i]);
        const int y2 = round_clamp_parity(val + ((val >= 0) ? eps : -eps));
        int u = (y2 + y2_max) / 2;
        u = clamp_int(u, 0, y2_max);
        code[i] = static_cast<uint8_t>(u);
    }
    double sum_y2 = 0.0;
    for (size_t i = 0; i < dim; ++i) {
        const double y = static_cast<double>(code[i]) - c;
        sum_y2 += y * y;
    }
    *y_norm = static_cast<float>(std::sqrt(sum_y2));
    if (!std::isfinite(*y_norm) || *y_norm <= 0.0F) {
        *y_norm = 1.0F;
    }
}

// RaBitQuantizer::PackIntoPlanes (rabitq_quantizer.cpp:431-453), planes in logical order (no split storage).
inline void
rabitq_pack_planes(const uint8_t* scalar, uint64_t dim, int bits, uint8_t* planes) {
    const uint64_t plane_bytes = (dim + 7) / 8;
    std::memset(planes, 0, plane_bytes * bits);
    for (uint64_t i = 0; i < dim; ++i) {
        for (int b = 0; b < bits; ++b) {
            if ((scalar[i] >> b) & 1U) {
                planes[b * plane_bytes + (i >> 3)] |= static_cast<uint8_t>(1U << (i & 7));
            }
        }
    }
}

inline float
rd_f32(const uint8_t* p) {
    float v;
    std::memcpy(&v, p, 4);
    return v;
}
inline void
wr_f32(uint8_t* p, float v) {
    std::memcpy(p, &v, 4);
}

// y = Q x, Q row-major (random_orthogonal_transformer.cpp:58-77; cblas_sgemv RowMajor NoTrans).
inline void
rotate(const float* rot, const float* x, float* y, uint64_t dim) {
    for (uint64_t i = 0; i < dim; ++i) {
        y[i] = fp32_ip(rot + i * dim, x, dim);
    }
}

// rabitq_quantizer.cpp:915-939
inline float
l2_ube(float nb, float nq, float est_ip_norm) {
    float p1 = nb * nb;
    float p2 = nq * nq;
    float p3 = -2 * nb * nq * est_ip_norm;
    return p1 + p2 + p3;
}

inline float
recover_sq4u(uint32_t ip, float base_sum, float query_sum, float lb, float delta, float inv_sqrt_d,
             uint64_t dim) {
    float p1 = inv_sqrt_d * delta * 2 * static_cast<float>(ip);
    float p2 = inv_sqrt_d * lb * 2 * base_sum;
    float p3 = inv_sqrt_d * delta * query_sum;
    float p4 = inv_sqrt_d * lb * static_cast<float>(dim);
    return p1 + p2 - p3 - p4;
}

// ---------------------------------------------------------------- product quantization, fast-scan form (pqfs)
// pq_fastscan_quantizer.cpp: pq_dim subspaces of dim / pq_dim dimensions, 16 centroids each
// (codebooks[subspace][centroid][subspace_dim], :117-122 of the header); a code is one 4-bit centroid index per
// subspace, subspace i in byte i / 2, low nibble for even i (:97-127).
constexpr uint64_t kPqCentroids = 16;

inline uint8_t
pq_nibble(const uint8_t* code, uint64_t i) {
    return (i & 1) ? static_cast<uint8_t>(code[i >> 1] >> 4) : static_cast<uint8_t>(code[i >> 1] & 0x0F);
}

// EncodeOneImpl (pq_fastscan_quantizer.cpp:97-127): per subspace the first centroid of smallest FP32ComputeL2Sqr
// (strict <, starting from FLT_MAX); cosine normalises the row first.
inline void
pq_encode_one(const float* x, uint64_t dim, uint64_t pq_dim, const float* codebooks, int metric, uint8_t* code) {
    const uint64_t sd = dim / pq_dim;
    std::vector<float> tmp;
    const float* cur = x;
    if (metric == kCosine) {
        tmp.resize(dim);
        normalize(x, tmp.data(), dim);
        cur = tmp.data();
    }
    std::memset(code, 0, (pq_dim + 1) / 2);
    for (uint64_t i = 0; i < pq_dim; ++i) {
        float nearest = std::numeric_limits<float>::max();
        uint8_t id = 0;
        const float* base = codebooks + i * sd * kPqCentroids;
        for (uint64_t j = 0; j < kPqCentroids; ++j) {
            float dist = fp32_l2sqr(cur + i * sd, base + j * sd, sd);
            if (dist < nearest) {
                nearest = dist;
                id = static_cast<uint8_t>(j);
            }
        }
        code[i / 2] |= (i & 1) ? static_cast<uint8_t>(id << 4) : id;
    }
}

// ProcessQueryImpl (pq_fastscan_quantizer.cpp:299-361): the float table lut[i][j] = FP32ComputeL2Sqr(sub-query i,
// centroid j) (l2) or their inner product (ip, cosine: the reference takes it from cblas_sgemv, whose order of
// summation is the library's; here in element order), quantised to bytes between its own smallest and largest
// entry (ScalarQuantizationTrainer::TrainUniform, CLASSIC: scalar_quantization_trainer.cpp:47-61,72-86):
// byte = uint8((v - lower) / diff * 255).  Output: pq_dim * 16 bytes, then diff and lower as floats.
inline void
pqfs_process_query(const float* q, uint64_t dim, uint64_t pq_dim, const float* codebooks, int metric, uint8_t* out) {
    const uint64_t sd = dim / pq_dim;
    std::vector<float> tmp;
    const float* cur = q;
    if (metric == kCosine) {
        tmp.resize(dim);
        normalize(q, tmp.data(), dim);
        cur = tmp.data();
    }
    std::vector<float> lut(pq_dim * kPqCentroids);
    for (uint64_t i = 0; i < pq_dim; ++i) {
        for (uint64_t j = 0; j < kPqCentroids; ++j) {
            const float* c = codebooks + (i * kPqCentroids + j) * sd;
            lut[i * kPqCentroids + j] = metric == kL2 ? fp32_l2sqr(cur + i * sd, c, sd) : fp32_ip(c, cur + i * sd, sd);
        }
    }
    float upper = std::numeric_limits<float>::lowest();
    float lower = std::numeric_limits<float>::max();
    for (float v : lut) {
        upper = std::max(upper, v);
        lower = std::min(lower, v);
    }
    const float diff = upper - lower;
    for (uint64_t j = 0; j < pq_dim * kPqCentroids; ++j) {
        // a float converted to uint8_t as the reference's assignment does; 0 / 0 (every entry equal) gives 0 here
        const float v = (lut[j] - lower) / diff * 255;
        out[j] = v == v ? static_cast<uint8_t>(static_cast<int32_t>(v)) : 0;
    }
    wr_f32(out + pq_dim * kPqCentroids, diff);
    wr_f32(out + pq_dim * kPqCentroids + 4, lower);
}

// The 32 codes of a block in the fast-scan order (pq_fastscan_quantizer.h:115-118, .cpp:241-266): subspace i takes 16
// bytes; byte j / 2 holds the code of vector MAPPER[j] in its low (even j) or high (odd j) nibble.
constexpr int32_t kPqMapper[32] = {0, 16, 8, 24, 1, 17, 9, 25, 2, 18, 10, 26, 3, 19, 11, 27,
                                   4, 20, 12, 28, 5, 21, 13, 29, 6, 22, 14, 30, 7, 23, 15, 31};

inline void
pqfs_package32(const uint8_t* codes, uint64_t pq_dim, int64_t valid, uint8_t* packaged) {
    const uint64_t cs = (pq_dim + 1) / 2;
    if (valid < 0) {
        valid = 32;
    }
    std::memset(packaged, 0, cs * 32);
    for (uint64_t i = 0; i < pq_dim; ++i) {
        for (int j = 0; j < 32; ++j) {
            const int v = kPqMapper[j];
            uint8_t code = v >= valid ? 0 : pq_nibble(codes + v * cs, i);
            packaged[i * 16 + j / 2] |= (j & 1) ? static_cast<uint8_t>(code << 4) : code;
        }
    }
}

inline void
pqfs_unpack32(const uint8_t* packaged, uint64_t pq_dim, uint8_t* codes) {
    const uint64_t cs = (pq_dim + 1) / 2;
    for (uint64_t i = 0; i < pq_dim; ++i) {
        for (int j = 0; j < 32; ++j) {
            const uint8_t byte = packaged[i * 16 + j / 2];
            const uint8_t code = (j & 1) ? static_cast<uint8_t>(byte >> 4) : static_cast<uint8_t>(byte & 0x0F);
            uint8_t* dst = codes + kPqMapper[j] * cs + i / 2;
            *dst = (i & 1) ? static_cast<uint8_t>((*dst & 0x0F) | (code << 4)) : static_cast<uint8_t>((*dst & 0xF0) | code);
        }
    }
}

// generic::PQFastScanLookUp32 (src/simd/generic.cpp:902-921): adds to result[32] the table bytes of the 32 packaged
// codes, subspace by subspace.
inline void
pqfs_lookup32(const uint8_t* lut, const uint8_t* packaged, uint64_t pq_dim, int32_t* result) {
    for (uint64_t i = 0; i < pq_dim; ++i) {
        const uint8_t* dict = lut + 16 * i;
        const uint8_t* code = packaged + 16 * i;
        for (uint64_t j = 0; j < 16; ++j) {
            if (j % 2 == 0) {
                result[j / 2] += dict[code[j] & 0x0F];
                result[16 + j / 2] += dict[code[j] >> 4];
            } else {
                result[8 + j / 2] += dict[code[j] & 0x0F];
                result[24 + j / 2] += dict[code[j] >> 4];
            }
        }
    }
}

// ScanBatchDistImpl's map (pq_fastscan_quantizer.cpp:166-199): int32 sum -> float(sum) / 255 * diff + lower, and
// 1 - that for ip / cosine.
inline float
pqfs_map(int32_t sum, float diff, float lower, int metric) {
    float v = static_cast<float>(sum) / 255.0F * diff + lower;
    return metric == kL2 ? v : 1.0F - v;
}

// One processed query against one code in the plain (not packaged) layout: the sum PQFastScanLookUp32 forms for
// that vector, mapped as above.
inline float
pqfs_dist(const uint8_t* q, const uint8_t* code, uint64_t pq_dim, int metric) {
    int32_t sum = 0;
    for (uint64_t i = 0; i < pq_dim; ++i) {
        sum += q[16 * i + pq_nibble(code, i)];
    }
    return pqfs_map(sum, rd_f32(q + pq_dim * kPqCentroids), rd_f32(q + pq_dim * kPqCentroids + 4), metric);
}

// ---------------------------------------------------------------- the reference's compiled kernels (timing only)
// When oracle/_ref is built, a benchmark's CPU leg can put the reference's own SIMD kernels (vsag::<isa>::*) under
// the loops restated below, through orc_set_reference_kernels.  All null by default: parity checks always run the
// scalar restatements above.
struct RefKernels {
    float (*fp32_l2)(const float*, const float*, uint64_t) = nullptr;
    float (*fp32_ip)(const float*, const float*, uint64_t) = nullptr;
    float (*sq4u_ip)(const uint8_t*, const uint8_t*, uint64_t) = nullptr;
    float (*sq8u_ip)(const uint8_t*, const uint8_t*, uint64_t) = nullptr;
    uint32_t (*rabitq_sq4u_ip)(const uint8_t*, const uint8_t*, uint64_t) = nullptr;
};
RefKernels g_ref;

// ---------------------------------------------------------------- bounded heaps
using Rec = std::pair<float, uint32_t>;
struct CmpMax {
    bool
    operator()(const Rec& a, const Rec& b) const {
        return a.first < b.first;
    }
};

// impl/heap/standard_heap.cpp:24-53 (max_heap, fixed_size): when full, dist > top is dropped,
// dist == top is pushed and one maximum popped.
struct FixedMaxHeap {
    std::vector<Rec> q;
    uint64_t cap;
    explicit FixedMaxHeap(uint64_t k) : cap(k) {
        q.reserve(k + 1);
    }
    void
    push(float d, uint32_t id) {
        if (q.size() == cap && !q.empty()) {
            if (d > q.front().first) {
                return;
            }
        }
        q.emplace_back(d, id);
        std::push_heap(q.begin(), q.end(), CmpMax());
        if (q.size() > cap) {
            pop();
        }
    }
    void
    pop() {
        std::pop_heap(q.begin(), q.end(), CmpMax());
        q.pop_back();
    }
    // inner_index_interface.cpp:1141-1145: pop into slots count-1 .. 0 -> ascending.
    uint64_t
    drain(uint32_t* ids, float* dists) {
        uint64_t n = q.size();
        for (int64_t j = static_cast<int64_t>(n) - 1; j >= 0; --j) {
            dists[j] = q.front().first;
            ids[j] = q.front().second;
            pop();
        }
        return n;
    }
};

// algorithm/ivf/flat_bucket_searcher.cpp:62-104 and impl/reorder/flatten_reorder.cpp:99-110: push only
// when the heap is not full or dist < cached top (strict), then pop down to topk.
struct StrictMaxHeap {
    std::vector<Rec> q;
    uint64_t cap;
    float top = std::numeric_limits<float>::max();
    explicit StrictMaxHeap(uint64_t k) : cap(k) {
        q.reserve(k + 1);
    }
    void
    push(float d, uint32_t id) {
        if (q.size() < cap || d < top) {
            q.emplace_back(d, id);
            std::push_heap(q.begin(), q.end(), CmpMax());
        }
        while (q.size() > cap) {
            std::pop_heap(q.begin(), q.end(), CmpMax());
            q.pop_back();
        }
        if (!q.empty() && q.size() == cap) {
            top = q.front().first;
        }
    }
    uint64_t
    drain(uint32_t* ids, float* dists) {
        uint64_t n = q.size();
        for (int64_t j = static_cast<int64_t>(n) - 1; j >= 0; --j) {
            dists[j] = q.front().first;
            ids[j] = q.front().second;
            std::pop_heap(q.begin(), q.end(), CmpMax());
            q.pop_back();
        }
        return n;
    }
};

// One (query, code) distance of the chosen store kind, as the quantizers' ComputeDistImpl return it:
// L2 -> squared L2, IP/cosine -> 1 - ip (fp32_quantizer.cpp:164-188, scalar_quantizer.cpp:180-196).
enum Kind { kFP32 = 0, kSQ8 = 1, kSQ4 = 2, kSQ4U = 3, kSQ8U = 4, kRaBitQ = 5, kPQFS = 6 };

struct Store {
    int kind;
    int metric;
    uint64_t dim;
    uint64_t code_size;
    const uint8_t* codes;
    const float* lb;    // per-dim (sq8/sq4) or &scalar (uniform)
    const float* diff;  // per-dim (sq8/sq4) or &scalar (uniform)
    int query_bits;     // rabitq only
};

inline float
uniform_dist(const Store& s, const uint8_t* qcode, const uint8_t* code) {
    // sq4_uniform_quantizer.cpp:166-201 ; sq8_uniform_quantizer.cpp:141-170
    int bits = s.kind == kSQ4U ? 4 : 8;
    UniformLayout l = uniform_layout(s.dim, bits, s.metric);
    float levels = bits == 4 ? 15.0F : 255.0F;
    float diff = *s.diff;
    float lb = *s.lb;
    float scalar_rate = static_cast<float>((diff / static_cast<double>(levels)) * (diff / static_cast<double>(levels)));
    float result;
    if (bits == 4) {
        result = g_ref.sq4u_ip ? g_ref.sq4u_ip(qcode, code, s.dim) : static_cast<float>(sq4u_codes_ip(qcode, code, s.dim));
    } else {
        result = g_ref.sq8u_ip ? g_ref.sq8u_ip(qcode, code, s.dim) : static_cast<float>(sq8u_codes_ip(qcode, code, s.dim));
    }
    if (s.metric == kL2) {
        uint64_t n1, n2;
        std::memcpy(&n1, qcode + l.offset_norm, 8);
        std::memcpy(&n2, code + l.offset_norm, 8);
        return (static_cast<float>(n1) + static_cast<float>(n2) - 2 * result) * scalar_rate;
    }
    float s1 = rd_f32(qcode + l.offset_sum);
    float s2 = rd_f32(code + l.offset_sum);
    result = lb * (s1 + s2) + scalar_rate * result + lb * lb;
    return 1 - result;
}

// rabitq_quantizer.cpp:1775-1860: 1-bit base with a 4-bit or 32-bit query, multi-bit base with a 32-bit query.
inline float
rabitq_dist(const RabitqLayout& l, int metric, int query_bits, const uint8_t* qcode, const uint8_t* code) {
    float inv_sqrt_d = 1.0F / std::sqrt(static_cast<float>(l.dim));
    float ip_bq;
    query_bits &= 255;
    if (l.base_bits != 1) {
        const float query_raw_sum = rd_f32(qcode + l.q_offset_sum);
        const float ip_yu_q = rabitq_float_planes_ip(reinterpret_cast<const float*>(qcode), code, l.dim, l.base_bits);
        ip_bq = ip_obar_q(ip_yu_q, query_raw_sum, rd_f32(code + l.offset_norm_code), l.base_bits);
    } else if (query_bits == 4) {
        std::vector<uint8_t> tmp(l.aligned_dim / 8, 0);
        std::memcpy(tmp.data(), code, l.offset_norm);
        uint32_t ip = g_ref.rabitq_sq4u_ip ? g_ref.rabitq_sq4u_ip(qcode, tmp.data(), l.aligned_dim)
                                           : rabitq_sq4u_binary_ip(qcode, tmp.data(), l.aligned_dim);
        float base_sum = rd_f32(code + l.offset_sum);
        float query_sum = rd_f32(qcode + l.q_offset_sum);
        float lb = rd_f32(qcode + l.q_offset_lb);
        float delta = rd_f32(qcode + l.q_offset_delta);
        ip_bq = recover_sq4u(ip, base_sum, query_sum, lb, delta, inv_sqrt_d, l.dim);
    } else {
        ip_bq = rabitq_float_binary_ip(reinterpret_cast<const float*>(qcode), code, l.dim, inv_sqrt_d);
    }
    float query_norm = rd_f32(qcode + l.q_offset_norm);
    float base_norm = rd_f32(code + l.offset_norm);
    float query_raw_norm = 0, base_raw_norm = 0;
    if (l.has_raw_norm) {
        query_raw_norm = rd_f32(qcode + l.q_offset_raw_norm);
        base_raw_norm = rd_f32(code + l.offset_raw_norm);
    }
    float base_error = rd_f32(code + l.offset_error);
    if (std::abs(base_error) < 1e-5) {
        base_error = (base_error >= 0) ? 1.0F : -1.0F;
    }
    float ip_est = ip_bq / base_error;
    float result = l2_ube(base_norm, query_norm, ip_est);
    auto approx_zero = [](float v) { return std::abs(v) < 1e-5; };
    if (metric == kCosine) {
        if (approx_zero(query_raw_norm) || approx_zero(base_raw_norm)) {
            result = 1;
        } else {
            result = 1 - (query_raw_norm * query_raw_norm + base_raw_norm * base_raw_norm - result) * 0.5F /
                             (query_raw_norm * base_raw_norm);
        }
    }
    if (metric == kIP) {
        if (approx_zero(query_raw_norm) || approx_zero(base_raw_norm)) {
            result = 1;
        } else {
            result = 1 - (query_raw_norm * query_raw_norm + base_raw_norm * base_raw_norm - result) * 0.5F;
        }
    }
    return result;
}

inline float
store_dist(const Store& s, const RabitqLayout* rl, const uint8_t* q, const uint8_t* code) {
    const float* qf = reinterpret_cast<const float*>(q);
    switch (s.kind) {
        case kFP32: {
            const float* x = reinterpret_cast<const float*>(code);
            if (s.metric == kL2) {
                return g_ref.fp32_l2 ? g_ref.fp32_l2(qf, x, s.dim) : fp32_l2sqr(qf, x, s.dim);
            }
            return 1 - (g_ref.fp32_ip ? g_ref.fp32_ip(qf, x, s.dim) : fp32_ip(qf, x, s.dim));
        }
        case kSQ8:
            return s.metric == kL2 ? sq8_l2sqr(qf, code, s.lb, s.diff, s.dim)
                                   : 1 - sq8_ip(qf, code, s.lb, s.diff, s.dim);
        case kSQ4:
            return s.metric == kL2 ? sq4_l2sqr(qf, code, s.lb, s.diff, s.dim)
                                   : 1 - sq4_ip(qf, code, s.lb, s.diff, s.dim);
        case kSQ4U:
        case kSQ8U:
            return uniform_dist(s, q, code);
        case kRaBitQ:
            return rabitq_dist(*rl, s.metric, s.query_bits, q, code);
        case kPQFS:
            return pqfs_dist(q, code, s.dim, s.metric);  // s.dim: the number of subspaces
    }
    return 0;
}

}  // namespace

// ================================================================= exported C entry points

// Puts compiled kernels of the reference (addresses of vsag::<isa>::FP32ComputeL2Sqr, FP32ComputeIP,
// SQ4UniformComputeCodesIP, SQ8UniformComputeCodesIP, RaBitQSQ4UBinaryIP; null = keep the restatement) under the
// scan loops of this file.  For timing the CPU baseline only; call with all nulls to go back.
ORC_API void
orc_set_reference_kernels(void* fp32_l2, void* fp32_ip, void* sq4u_ip, void* sq8u_ip, void* rabitq_sq4u_ip) {
    g_ref.fp32_l2 = reinterpret_cast<decltype(g_ref.fp32_l2)>(fp32_l2);
    g_ref.fp32_ip = reinterpret_cast<decltype(g_ref.fp32_ip)>(fp32_ip);
    g_ref.sq4u_ip = reinterpret_cast<decltype(g_ref.sq4u_ip)>(sq4u_ip);
    g_ref.sq8u_ip = reinterpret_cast<decltype(g_ref.sq8u_ip)>(sq8u_ip);
    g_ref.rabitq_sq4u_ip = reinterpret_cast<decltype(g_ref.rabitq_sq4u_ip)>(rabitq_sq4u_ip);
}

// Threads of the OpenMP loops below (0 = leave as is); the loops that take a `threads` argument set it themselves.
ORC_API void
orc_set_threads(int threads) {
    if (threads > 0) {
        omp_set_num_threads(threads);
    }
}

ORC_API float
orc_fp32_l2sqr(const float* q, const float* x, uint64_t dim) {
    return fp32_l2sqr(q, x, dim);
}
ORC_API float
orc_fp32_ip(const float* q, const float* x, uint64_t dim) {
    return fp32_ip(q, x, dim);
}
ORC_API float
orc_normalize(const float* from, float* to, uint64_t dim) {
    return normalize(from, to, dim);
}
ORC_API float
orc_normalize_with_centroid(const float* from, const float* c, float* to, uint64_t dim) {
    return normalize_with_centroid(from, c, to, dim);
}
ORC_API float
orc_sq8_ip(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    return sq8_ip(q, c, lb, diff, dim);
}
ORC_API float
orc_sq8_l2sqr(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    return sq8_l2sqr(q, c, lb, diff, dim);
}
ORC_API float
orc_sq4_ip(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    return sq4_ip(q, c, lb, diff, dim);
}
ORC_API float
orc_sq4_l2sqr(const float* q, const uint8_t* c, const float* lb, const float* diff, uint64_t dim) {
    return sq4_l2sqr(q, c, lb, diff, dim);
}
ORC_API int32_t
orc_sq4u_codes_ip(const uint8_t* a, const uint8_t* b, uint64_t dim) {
    return sq4u_codes_ip(a, b, dim);
}
ORC_API int32_t
orc_sq8u_codes_ip(const uint8_t* a, const uint8_t* b, uint64_t dim) {
    return sq8u_codes_ip(a, b, dim);
}
ORC_API uint32_t
orc_rabitq_sq4u_binary_ip(const uint8_t* planes, const uint8_t* bits, uint64_t dim) {
    return rabitq_sq4u_binary_ip(planes, bits, dim);
}
ORC_API float
orc_rabitq_float_binary_ip(const float* v, const uint8_t* bits, uint64_t dim, float inv_sqrt_d) {
    return rabitq_float_binary_ip(v, bits, dim, inv_sqrt_d);
}

// ---- scalar-quantization trainer --------------------------------------------------------------
// scalar_quantization_trainer.cpp:125-146: deterministic strided sample, at most max_sample rows.
static uint64_t
sq_sample(const float* data, uint64_t count, uint64_t dim, bool need_normalize, uint64_t max_sample,
          std::vector<float>& out) {
    uint64_t step = 2147483647UL % count;
    uint64_t sample_count = max_sample;
    if (count <= max_sample) {
        step = 1;
        sample_count = count;
    }
    out.resize(sample_count * dim);
    for (uint64_t j = 0; j < sample_count; ++j) {
        uint64_t idx = (j * step) % count;
        if (need_normalize) {
            normalize(data + idx * dim, out.data() + j * dim, dim);
        } else {
            std::memcpy(out.data() + j * dim, data + idx * dim, dim * sizeof(float));
        }
    }
    return sample_count;
}

// scalar_quantization_trainer.cpp:72-122.  mode 1 = CLASSIC (min/max), 3 = TRUNC_BOUND (the default):
// two bounded heaps per dimension, seeded with a sentinel, keep the ignore_count largest / smallest.
static void
sq_train_bounds(const float* s, uint64_t count, uint64_t dim, int bits, float trunc_rate, int mode, float* upper,
                float* lower) {
    if (mode == 1) {
        for (uint64_t i = 0; i < dim; ++i) {
            upper[i] = std::numeric_limits<float>::lowest();
            lower[i] = std::numeric_limits<float>::max();
            for (uint64_t j = 0; j < count; ++j) {
                float v = s[j * dim + i];
                upper[i] = std::max(upper[i], v);
                lower[i] = std::min(lower[i], v);
            }
        }
        return;
    }
    double ignore_rate = 0.001;
    if (bits == 4) {
        ignore_rate = trunc_rate;
    }
    auto ignore_count = static_cast<uint64_t>(static_cast<double>(count - 1) * ignore_rate);
    ignore_count = ignore_count < 1 ? 1 : ignore_count;
    for (uint64_t i = 0; i < dim; ++i) {
        std::priority_queue<float, std::vector<float>, std::greater<>> heap_max;
        std::priority_queue<float, std::vector<float>, std::less<>> heap_min;
        heap_max.emplace(std::numeric_limits<float>::lowest());
        heap_min.emplace(std::numeric_limits<float>::max());
        for (uint64_t j = 0; j < count; ++j) {
            float v = s[j * dim + i];
            if (v > heap_max.top() || heap_max.size() < ignore_count) {
                heap_max.emplace(v);
            }
            if (heap_max.size() > ignore_count) {
                heap_max.pop();
            }
            if (v < heap_min.top() || heap_min.size() < ignore_count) {
                heap_min.emplace(v);
            }
            if (heap_min.size() > ignore_count) {
                heap_min.pop();
            }
        }
        upper[i] = heap_max.top();
        lower[i] = heap_min.top();
    }
}

// ScalarQuantizationTrainer::Train (scalar_quantization_trainer.cpp:30-45) + ScalarQuantizer::TrainImpl
// (scalar_quantizer.cpp:52-73): returns lower_bound[d] and diff[d] = upper - lower.
ORC_API void
orc_sq_train(const float* data, uint64_t count, uint64_t dim, int bits, int metric, int mode, float trunc_rate,
             uint64_t max_sample, float* lb, float* diff) {
    std::vector<float> sample;
    uint64_t sc = sq_sample(data, count, dim, metric == kCosine, max_sample ? max_sample : 100000, sample);
    sq_train_bounds(sample.data(), sc, dim, bits, trunc_rate, mode, diff, lb);
    for (uint64_t i = 0; i < dim; ++i) {
        diff[i] -= lb[i];
    }
}

// ScalarQuantizationTrainer::TrainUniform (scalar_quantization_trainer.cpp:47-70) + the uniform
// quantizers' TrainImpl (sq4_uniform_quantizer.cpp:86-108: TRUNC_BOUND; sq8_uniform_quantizer.cpp:76-98:
// CLASSIC).  Returns scalar lower bound and diff.
ORC_API void
orc_sq_train_uniform(const float* data, uint64_t count, uint64_t dim, int bits, int metric, int mode, float trunc_rate,
                     uint64_t max_sample, float* lb_out, float* diff_out) {
    std::vector<float> sample;
    uint64_t sc = sq_sample(data, count, dim, metric == kCosine, max_sample ? max_sample : 100000, sample);
    std::vector<float> upper(dim), lower(dim);
    sq_train_bounds(sample.data(), sc, dim, bits, trunc_rate, mode, upper.data(), lower.data());
    float ub, lb;
    if (mode == 1) {
        ub = *std::max_element(upper.begin(), upper.end());
        lb = *std::min_element(lower.begin(), lower.end());
    } else {
        ub = *std::min_element(upper.begin(), upper.end());
        lb = *std::max_element(lower.begin(), lower.end());
        if (lb > ub) {
            std::swap(lb, ub);
        }
    }
    *lb_out = lb;
    *diff_out = ub - lb;
}

// ScalarQuantizer::EncodeOneImpl (scalar_quantizer.cpp:85-112): divide by diff[d], clamp, truncate.
ORC_API void
orc_sq_encode(const float* data, uint64_t n, uint64_t dim, int bits, int metric, const float* lb, const float* diff,
              uint8_t* codes) {
    uint64_t code_size = align_up(dim * bits, 8) / 8;
    float levels = static_cast<float>((1 << bits) - 1);
    std::vector<float> tmp(dim);
    for (uint64_t i = 0; i < n; ++i) {
        const float* cur = data + i * dim;
        if (metric == kCosine) {
            normalize(cur, tmp.data(), dim);
            cur = tmp.data();
        }
        uint8_t* c = codes + i * code_size;
        std::memset(c, 0, code_size);
        for (uint64_t d = 0; d < dim; ++d) {
            float delta;
            if (diff[d] < std::numeric_limits<float>::epsilon()) {
                delta = 1.0F;
            } else {
                delta = 1.0F * (cur[d] - lb[d]) / diff[d];
            }
            delta = clamp_delta(delta);
            auto scaled = static_cast<uint8_t>(levels * delta);
            uint64_t idx = (d * bits) / 8;
            uint64_t off = (d * bits) % 8;
            c[idx] |= scaled << off;
        }
    }
}

// ScalarQuantizer::DecodeOneImpl (scalar_quantizer.cpp:114-125).
ORC_API void
orc_sq_decode(const uint8_t* codes, uint64_t n, uint64_t dim, int bits, const float* lb, const float* diff,
              float* data) {
    uint64_t code_size = align_up(dim * bits, 8) / 8;
    float levels = static_cast<float>(1 << bits) - 1.0F;
    for (uint64_t i = 0; i < n; ++i) {
        for (uint64_t d = 0; d < dim; ++d) {
            uint64_t idx = (d * bits) / 8, off = (d * bits) % 8;
            data[i * dim + d] =
                static_cast<float>((codes[i * code_size + idx] >> off) & ((1 << bits) - 1)) / levels * diff[d] + lb[d];
        }
    }
}

ORC_API uint64_t
orc_squ_code_size(uint64_t dim, int bits, int metric) {
    return uniform_layout(dim, bits, metric).code_size;
}

// SQ4UniformQuantizer::EncodeOneImpl (sq4_uniform_quantizer.cpp:110-152) and SQ8UniformQuantizer::
// EncodeOneImpl (sq8_uniform_quantizer.cpp:100-132): multiply by 1/diff, clamp, truncate.  Padding
// bytes (which the reference leaves untouched) are written as zero.
ORC_API void
orc_squ_encode(const float* data, uint64_t n, uint64_t dim, int bits, int metric, float lb, float diff,
               uint8_t* codes) {
    UniformLayout l = uniform_layout(dim, bits, metric);
    float levels = bits == 4 ? 15.0F : 255.0F;
    std::vector<float> tmp(dim);
    float inv_diff = diff == 0.0F ? 0.0F : 1.0F / diff;
    for (uint64_t i = 0; i < n; ++i) {
        const float* cur = data + i * dim;
        if (metric == kCosine) {
            normalize(cur, tmp.data(), dim);
            cur = tmp.data();
        }
        uint8_t* c = codes + i * l.code_size;
        std::memset(c, 0, l.code_size);
        uint64_t norm = 0;
        float sum = 0, codes_sum = 0;
        for (uint64_t d = 0; d < dim; ++d) {
            float delta = (cur[d] - lb) * inv_diff;
            delta = clamp_delta(delta);
            auto scaled = static_cast<uint8_t>(levels * delta);
            if (bits == 4) {
                if (d & 1) {
                    c[d >> 1] |= scaled << 4;
                } else {
                    c[d >> 1] = scaled;
                }
            } else {
                c[d] = scaled;
            }
            norm += static_cast<uint64_t>(scaled) * static_cast<uint64_t>(scaled);
            sum += cur[d];
            codes_sum += static_cast<float>(scaled);
        }
        if (metric == kL2) {
            std::memcpy(c + l.offset_norm, &norm, 8);
        }
        if (l.has_sum) {
            wr_f32(c + l.offset_sum, sum);
            if (l.has_codes_sum) {
                wr_f32(c + l.offset_codes_sum, codes_sum);
            }
        }
    }
}

ORC_API float
orc_squ_dist(const uint8_t* qcode, const uint8_t* code, uint64_t dim, int bits, int metric, float lb, float diff) {
    Store s{bits == 4 ? kSQ4U : kSQ8U, metric, dim, 0, nullptr, &lb, &diff, 0};
    return uniform_dist(s, qcode, code);
}

// ---- RaBitQ -----------------------------------------------------------------------------------
ORC_API uint64_t
orc_rabitq_code_size(uint64_t dim, int metric, int query_bits) {
    return rabitq_layout(dim, metric, query_bits).code_size;
}
ORC_API uint64_t
orc_rabitq_query_code_size(uint64_t dim, int metric, int query_bits) {
    return rabitq_layout(dim, metric, query_bits).query_code_size;
}

// RaBitQuantizer::TrainImpl (rabitq_quantizer.cpp:209-254): centroid = rotation applied to the
// fp32 running-sum mean of the data.  The rotation itself is an input (the reference draws it from
// std::random_device, random_orthogonal_transformer.cpp:101-102).
ORC_API void
orc_rabitq_train(const float* data, uint64_t n, uint64_t dim, const float* rot, float* centroid) {
    std::vector<float> mean(dim, 0.0F);
    for (uint64_t i = 0; i < n; ++i) {
        for (uint64_t d = 0; d < dim; ++d) {
            mean[d] += data[i * dim + d];
        }
    }
    for (uint64_t d = 0; d < dim; ++d) {
        mean[d] = mean[d] / static_cast<float>(n);
    }
    rotate(rot, mean.data(), centroid, dim);
}

// RaBitQuantizer::EncodeOneInternal, 1-bit branch (rabitq_quantizer.cpp:724-856).
ORC_API void
orc_rabitq_encode(const float* data, uint64_t n, uint64_t dim, const float* rot, const float* centroid, int metric,
                  int query_bits, uint8_t* codes) {
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    float inv_sqrt_d = 1.0F / std::sqrt(static_cast<float>(dim));
#pragma omp parallel
    {
        std::vector<float> t(dim), nd(dim);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < static_cast<int64_t>(n); ++i) {
            const float* x = data + i * dim;
            uint8_t* c = codes + i * l.code_size;
            std::memset(c, 0, l.code_size);
            float raw_norm = 0;
            if (l.has_raw_norm) {
                for (uint64_t d = 0; d < dim; ++d) {
                    raw_norm += x[d] * x[d];
                }
            }
            raw_norm = std::sqrt(raw_norm);
            rotate(rot, x, t.data(), dim);
            float norm = normalize_with_centroid(t.data(), centroid, nd.data(), dim);
            uint64_t binary_sum = 0;
            for (uint64_t d = 0; d < dim; ++d) {
                if (nd[d] >= 0.0F) {
                    ++binary_sum;
                    c[d / 8] |= static_cast<uint8_t>(1U << (d % 8));
                }
            }
            float error = rabitq_float_binary_ip(nd.data(), c, dim, inv_sqrt_d);
            wr_f32(c + l.offset_norm, norm);
            wr_f32(c + l.offset_error, error);
            if (l.has_sum) {
                wr_f32(c + l.offset_sum, static_cast<float>(binary_sum));
            }
            if (l.has_raw_norm) {
                wr_f32(c + l.offset_raw_norm, raw_norm);
            }
        }
    }
}

// ---- FhtKacRotator (rabitq_use_fht) -----------------------------------------------------------------------
// The primitives of simd/generic.cpp:953-985 (FlipSign, VecRescale, FHTRotate over RotateOp of
// simd/kernels/butterfly.h:36-55, KacsWalk of butterfly.h:61-94).
static void
fht_flip_sign(const uint8_t* flip, float* data, uint64_t dim) {
    for (uint64_t i = 0; i < dim; ++i) {
        if ((flip[i / 8] & (1 << (i % 8))) != 0) {
            data[i] = -data[i];
        }
    }
}
static void
fht_rescale(float* data, uint64_t dim, float val) {
    for (uint64_t i = 0; i < dim; ++i) {
        data[i] *= val;
    }
}
static void
fht_rotate(float* data, uint64_t n) {
    for (uint64_t step = 1; step < n; step *= 2) {
        for (uint64_t i = 0; i < n; i += step * 2) {
            for (uint64_t j = 0; j < step; ++j) {
                const float g1 = data[i + j], g2 = data[i + j + step];
                data[i + j] = g1 + g2;
                data[i + j + step] = g1 - g2;
            }
        }
    }
}
static void
fht_kacs_walk(float* data, uint64_t len) {
    const uint64_t base = len % 2, offset = base + len / 2;
    for (uint64_t i = 0; i < len / 2; ++i) {
        const float x = data[i], y = data[i + offset];
        data[i] = x + y;
        data[i + offset] = x - y;
    }
    if (base != 0) {
        data[len / 2] *= std::sqrt(2.0F);
    }
}
ORC_API void
orc_fht_primitive(int which, const uint8_t* flip, float* data, uint64_t dim, float val) {
    switch (which) {
        case 0: fht_flip_sign(flip, data, dim); break;
        case 1: fht_rescale(data, dim, val); break;
        case 2: fht_rotate(data, dim); break;
        default: fht_kacs_walk(data, dim); break;
    }
}

// FhtKacRotator::Transform / InverseTransform (impl/transform/fht_kac_rotate_transformer.cpp:64-120): four rounds
// (ROUND, fht_kac_rotate_transformer.h:53) of sign flips (flip: 4 x ceil(dim / 8) bytes), a Hadamard transform of the
// leading power-of-two block and a rescale; other dimensions alternate the leading and the trailing block with a
// Kac walk in between and close with a factor 1/4.
ORC_API void
orc_fht_kac_transform(const uint8_t* flip, uint64_t dim, int inverse, const float* in, float* out) {
    const uint64_t flip_offset = (dim + 7) / 8;
    uint64_t trunc = 1;
    while (trunc * 2 <= dim) {
        trunc *= 2;
    }
    const float fac = 1.0F / std::sqrt(static_cast<float>(trunc));
    std::memcpy(out, in, dim * sizeof(float));
    const uint64_t start = dim - trunc;
    if (!inverse) {
        if (trunc == dim) {
            for (int t = 0; t < 4; ++t) {
                fht_flip_sign(flip + t * flip_offset, out, dim);
                fht_rotate(out, trunc);
                fht_rescale(out, trunc, fac);
            }
            return;
        }
        for (int t = 0; t < 4; t += 2) {
            fht_flip_sign(flip + t * flip_offset, out, dim);
            fht_rotate(out, trunc);
            fht_rescale(out, trunc, fac);
            fht_kacs_walk(out, dim);
            fht_flip_sign(flip + (t + 1) * flip_offset, out, dim);
            fht_rotate(out + start, trunc);
            fht_rescale(out + start, trunc, fac);
            fht_kacs_walk(out, dim);
        }
        fht_rescale(out, dim, 0.25F);
        return;
    }
    if (trunc == dim) {
        for (int t = 3; t >= 0; --t) {
            fht_rotate(out, trunc);
            fht_rescale(out, trunc, fac);
            fht_flip_sign(flip + t * flip_offset, out, dim);
        }
        return;
    }
    fht_rescale(out, dim, 0.25F);
    for (int t = 3; t > 0; t -= 2) {
        fht_kacs_walk(out, dim);
        fht_rotate(out + start, trunc);
        fht_rescale(out + start, trunc, fac);
        fht_flip_sign(flip + t * flip_offset, out, dim);
        fht_kacs_walk(out, dim);
        fht_rotate(out, trunc);
        fht_rescale(out, trunc, fac);
        fht_flip_sign(flip + (t - 1) * flip_offset, out, dim);
    }
}

// RaBitQuantizer::DecodeOneImpl (rabitq_quantizer.cpp:871-899), which use_residual needs for the l2 bias of a code
// (bucket_datacell.h:645-650): 1-bit codes only (other widths return false and write nothing: 0 here, rows left as
// they are).  The sign vector over sqrt(d), InverseNormalizeWithCentroid (simd/kernels/normalize.h:88-119:
// from * norm + centroid per element), then x = R^T y (RandomOrthogonalMatrix::InverseTransform,
// random_orthogonal_transformer.cpp:80-94: a row-major sgemv with Trans; summed over the rows in order here, BLAS
// leaves the order open).
ORC_API int
orc_rabitq_decode(const uint8_t* codes, uint64_t n, uint64_t dim, const float* rot, const float* centroid, int metric,
                  int query_bits, float* out) {
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    if (l.base_bits != 1) {
        return 0;
    }
    const float inv_sqrt_d = 1.0F / std::sqrt(static_cast<float>(dim));
#pragma omp parallel
    {
        std::vector<float> y(dim);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < static_cast<int64_t>(n); ++i) {
            const uint8_t* c = codes + i * l.code_size;
            const float norm = rd_f32(c + l.offset_norm);
            for (uint64_t d = 0; d < dim; ++d) {
                const bool bit = ((c[d / 8] >> (d % 8)) & 1) != 0;
                const float from = bit ? inv_sqrt_d : -inv_sqrt_d;
                y[d] = from * norm + centroid[d];
            }
            float* x = out + i * dim;
            for (uint64_t j = 0; j < dim; ++j) {
                float acc = 0.0F;
                for (uint64_t r = 0; r < dim; ++r) {
                    acc += rot[r * dim + j] * y[r];
                }
                x[j] = acc;
            }
        }
    }
    return 1;
}

// RaBitQuantizer::EncodeOneInternal, multi-bit branch (rabitq_quantizer.cpp:774-809): the scalar code of the rotated,
// centred, normalised row by FastEncodeRaBitQ or EncodeExtendRaBitQ, packed into bit planes; norm_code = |code - centre|,
// error = ip_obar_q(<o, code>, sum o, norm_code).  query_bits carries the base bits in its second byte.
ORC_API void
orc_rabitq_encode_multibit(const float* data, uint64_t n, uint64_t dim, const float* rot, const float* centroid,
                           int metric, int query_bits, int fast, uint64_t rounds, uint8_t* codes) {
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
#pragma omp parallel
    {
        std::vector<float> t(dim), nd(dim);
        std::vector<uint8_t> scalar(dim);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < static_cast<int64_t>(n); ++i) {
            const float* x = data + i * dim;
            uint8_t* c = codes + i * l.code_size;
            std::memset(c, 0, l.code_size);
            float raw_norm = 0;
            if (l.has_raw_norm) {
                for (uint64_t d = 0; d < dim; ++d) {
                    raw_norm += x[d] * x[d];
                }
            }
            raw_norm = std::sqrt(raw_norm);
            rotate(rot, x, t.data(), dim);
            float norm = normalize_with_centroid(t.data(), centroid, nd.data(), dim);
            float norm_code = 0;
            if (fast) {
                rabitq_fast_encode(nd.data(), dim, l.base_bits, rounds, scalar.data(), &norm_code);
            } else {
                rabitq_extend_encode(nd.data(), dim, l.base_bits, scalar.data(), &norm_code);
            }
            float query_sum = 0.0F;
            for (uint64_t d = 0; d < dim; ++d) {
                query_sum += nd[d];
            }
            rabitq_pack_planes(scalar.data(), dim, l.base_bits, c);
            wr_f32(c + l.offset_norm_code, norm_code);
            const float scalar_ip = rabitq_float_sq_ip(nd.data(), scalar.data(), dim);
            const float error = ip_obar_q(scalar_ip, query_sum, norm_code, l.base_bits);
            wr_f32(c + l.offset_norm, norm);
            wr_f32(c + l.offset_error, error);
            if (l.has_raw_norm) {
                wr_f32(c + l.offset_raw_norm, raw_norm);
            }
        }
    }
}

ORC_API void
orc_rabitq_fast_encode(const float* o, uint64_t dim, int bits, uint64_t rounds, uint8_t* code, float* y_norm) {
    rabitq_fast_encode(o, dim, bits, rounds, code, y_norm);
}
ORC_API void
orc_rabitq_extend_encode(const float* o, uint64_t dim, int bits, uint8_t* code, float* y_norm) {
    rabitq_extend_encode(o, dim, bits, code, y_norm);
}
ORC_API void
orc_rabitq_pack_planes(const uint8_t* scalar, uint64_t dim, int bits, uint8_t* planes) {
    rabitq_pack_planes(scalar, dim, bits, planes);
}
ORC_API float
orc_rabitq_float_planes_ip(const float* v, const uint8_t* planes, uint64_t dim, int bits) {
    return rabitq_float_planes_ip(v, planes, dim, bits);
}
ORC_API float
orc_rabitq_float_sq_ip(const float* v, const uint8_t* codes, uint64_t dim) {
    return rabitq_float_sq_ip(v, codes, dim);
}

// RaBitQuantizer::EncodeSQ + ReOrderSQ (rabitq_quantizer.cpp:2049-2088): per-query min/max, round to
// nearest of 15 levels, then bit b of every dim goes to plane b (planes aligned_dim/8 bytes apart).
ORC_API void
orc_rabitq_encode_sq(const float* normed, uint64_t dim, uint8_t* quantized, float* upper, float* lower, float* delta,
                     float* query_sum) {
    float lb = std::numeric_limits<float>::max();
    float ub = std::numeric_limits<float>::lowest();
    for (uint64_t i = 0; i < dim; ++i) {
        float v = normed[i];
        if (v < lb) {
            lb = v;
        }
        if (v > ub) {
            ub = v;
        }
    }
    float dl = (ub - lb) / 15;
    float inv_delta = (std::abs(dl) < 1e-5) ? 0.0F : 1.0F / dl;
    float qs = 0;
    for (uint64_t i = 0; i < dim; ++i) {
        auto val = std::round((normed[i] - lb) * inv_delta);
        quantized[i] = static_cast<uint8_t>(val);
        qs += static_cast<float>(val);
    }
    *upper = ub;
    *lower = lb;
    *delta = dl;
    *query_sum = qs;
}

ORC_API void
orc_rabitq_reorder_sq(const uint8_t* quantized, uint64_t dim, uint8_t* planes /* zeroed, 4*aligned_dim/8 */) {
    uint64_t offset = ((dim + 511) / 512 * 512) / 8;
    for (uint64_t d = 0; d < dim; ++d) {
        for (uint64_t b = 0; b < 4; ++b) {
            bool bit = (quantized[d] & (1 << b)) != 0;
            planes[b * offset + d / 8] |= (static_cast<int32_t>(bit) * (1 << (d % 8)));
        }
    }
}

// RaBitQuantizer::ProcessQueryImpl (rabitq_quantizer.cpp:2130-2217).
ORC_API void
orc_rabitq_process_query(const float* query, uint64_t dim, const float* rot, const float* centroid, int metric,
                         int query_bits, uint8_t* qcode) {
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    std::memset(qcode, 0, l.query_code_size);
    std::vector<float> t(dim), nd(dim);
    float raw = 0;
    if (l.has_raw_norm) {
        for (uint64_t d = 0; d < dim; ++d) {
            raw += query[d] * query[d];
        }
    }
    raw = std::sqrt(raw);
    rotate(rot, query, t.data(), dim);
    float qnorm = normalize_with_centroid(t.data(), centroid, nd.data(), dim);
    if ((query_bits & 255) == 4) {
        std::vector<uint8_t> quant(dim, 0);
        float ub, lb, delta, qsum;
        orc_rabitq_encode_sq(nd.data(), dim, quant.data(), &ub, &lb, &delta, &qsum);
        orc_rabitq_reorder_sq(quant.data(), dim, qcode);
        wr_f32(qcode + l.q_offset_lb, lb);
        wr_f32(qcode + l.q_offset_delta, delta);
        wr_f32(qcode + l.q_offset_sum, qsum);
    } else {
        std::memcpy(qcode, nd.data(), dim * sizeof(float));
    }
    if (l.base_bits != 1) {
        float query_raw_sum = 0;
        for (uint64_t d = 0; d < dim; ++d) {
            query_raw_sum += nd[d];
        }
        wr_f32(qcode + l.q_offset_sum, query_raw_sum);
    }
    wr_f32(qcode + l.q_offset_norm, qnorm);
    if (l.has_raw_norm) {
        wr_f32(qcode + l.q_offset_raw_norm, raw);
    }
}

ORC_API float
orc_rabitq_dist(const uint8_t* qcode, const uint8_t* code, uint64_t dim, int metric, int query_bits) {
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    return rabitq_dist(l, metric, query_bits, qcode, code);
}

// ---- k-means ----------------------------------------------------------------------------------
// KMeansCluster::find_nearest_one_with_blas (impl/cluster/kmeans_cluster.cpp:193-305).
// distances[m] = -2 <c_m, x> (the SGEMM; OpenBLAS 0.3.24 is absent, so the contraction is a plain fp32
// dot in element order), += y_sqr[m], first minimum, err += double(float(min + x_sqr)); returns err/n.
ORC_API double
orc_kmeans_assign(const float* x, uint64_t n, uint64_t dim, const float* cent, uint64_t k, int32_t* labels,
                  float* min_dist /* may be null: min_m(||c||^2 - 2<c,x>) */) {
    std::vector<float> y_sqr(k);
    for (uint64_t j = 0; j < k; ++j) {
        y_sqr[j] = fp32_ip(cent + j * dim, cent + j * dim, dim);
    }
    // Eight centroids side by side (ct[block][d][lane]) so that the compiler can run eight of the dot products
    // in one vector; every dot product is still the element-order fp32 sum of fp32_ip (multiply, then add).
    const uint64_t kb = (k + 7) / 8;
    std::vector<float> ct(kb * dim * 8, 0.0F);
    for (uint64_t j = 0; j < k; ++j) {
        for (uint64_t d = 0; d < dim; ++d) {
            ct[(j / 8) * dim * 8 + d * 8 + (j % 8)] = cent[j * dim + d];
        }
    }
    double error = 0.0;
    // Rows go four at a time through a block of centroids (the block stays in cache, four independent sums hide the
    // latency of the adds); the per-row results do not depend on the grouping.
    constexpr int R = 4;
    const int64_t ngroups = static_cast<int64_t>((n + R - 1) / R);
#pragma omp parallel
    {
        std::vector<float> dist(static_cast<size_t>(R) * kb * 8);
        double local = 0.0;
#pragma omp for schedule(static)
        for (int64_t g = 0; g < ngroups; ++g) {
            const uint64_t i0 = static_cast<uint64_t>(g) * R;
            const int rows = static_cast<int>(std::min<uint64_t>(R, n - i0));
            const float* xr[R];
            for (int r = 0; r < R; ++r) {
                xr[r] = x + (i0 + (r < rows ? r : 0)) * dim;
            }
            for (uint64_t b = 0; b < kb; ++b) {
                const float* cb = ct.data() + b * dim * 8;
                float acc[R][8];
                for (int r = 0; r < R; ++r) {
                    for (int l = 0; l < 8; ++l) {
                        acc[r][l] = 0.0F;
                    }
                }
                for (uint64_t d = 0; d < dim; ++d) {
                    for (int r = 0; r < R; ++r) {
                        const float xv = xr[r][d];
                        for (int l = 0; l < 8; ++l) {
                            acc[r][l] = cb[d * 8 + l] * xv + acc[r][l];
                        }
                    }
                }
                for (int r = 0; r < R; ++r) {
                    for (int l = 0; l < 8; ++l) {
                        dist[(r * kb + b) * 8 + l] = -2.0F * acc[r][l];
                    }
                }
            }
            for (int r = 0; r < rows; ++r) {
                float* dr = dist.data() + static_cast<size_t>(r) * kb * 8;
                for (uint64_t j = 0; j < k; ++j) {
                    dr[j] = 1.0F * y_sqr[j] + dr[j];
                }
                auto* me = std::min_element(dr, dr + k);
                const float* xi = xr[r];
                float x_sqr = fp32_ip(xi, xi, dim);
                labels[i0 + r] = static_cast<int32_t>(me - dr);
                if (min_dist != nullptr) {
                    min_dist[i0 + r] = *me;
                }
                local += static_cast<double>(*me + x_sqr);
            }
        }
#pragma omp critical
        error += local;
    }
    return error / static_cast<float>(n);
}

// Centroid update of KMeansCluster::Run (kmeans_cluster.cpp:108-172): fp32 sums of member rows in
// blocks of 1024 rows (merged here in block order; the reference merges in thread-completion order),
// scaled by 1/count.  Empty clusters are left untouched and reported through counts[j] == 0 (the
// reference re-seeds them from std::random_device, :156-171 — the caller does that with its own RNG).
ORC_API void
orc_kmeans_update(const float* x, const int32_t* labels, uint64_t n, uint64_t dim, uint64_t k, float* cent,
                  int32_t* counts) {
    std::vector<float> sums(k * dim, 0.0F), local(k * dim);
    std::vector<int32_t> lc(k);
    std::fill(counts, counts + k, 0);
    for (uint64_t s = 0; s < n; s += 1024) {
        uint64_t e = std::min(s + 1024, n);
        std::fill(local.begin(), local.end(), 0.0F);
        std::fill(lc.begin(), lc.end(), 0);
        for (uint64_t i = s; i < e; ++i) {
            int32_t l = labels[i];
            if (l >= 0 && l < static_cast<int32_t>(k)) {
                lc[l]++;
                for (uint64_t d = 0; d < dim; ++d) {
                    local[l * dim + d] += x[i * dim + d];
                }
            }
        }
        for (uint64_t j = 0; j < k; ++j) {
            if (lc[j] > 0) {
                counts[j] += lc[j];
                for (uint64_t d = 0; d < dim; ++d) {
                    sums[j * dim + d] += local[j * dim + d];
                }
            }
        }
    }
    for (uint64_t j = 0; j < k; ++j) {
        if (counts[j] > 0) {
            float inv = 1.0F / static_cast<float>(counts[j]);
            for (uint64_t d = 0; d < dim; ++d) {
                cent[j * dim + d] = sums[j * dim + d] * inv;
            }
        }
    }
}

// KMeansCluster::select_initial_centroids_kmeans_plus_plus (kmeans_cluster.cpp:383-435) with the random draws as
// inputs: `first` is what first_dis(gen) returned, draws[c - 1] in [0, 1) stands for the c-th prob_dis(gen) /
// total_weight (uniform_real_distribution<double>(0, w)(gen) = w * generate_canonical) or, when the total weight is 0,
// for dis(gen) / count.
ORC_API void
orc_kmeans_init_pp(const float* x, uint64_t n, uint64_t dim, uint64_t k, uint64_t first, const double* draws, float* cent,
                   uint64_t* picks) {
    std::memcpy(cent, x + first * dim, dim * sizeof(float));
    picks[0] = first;
    std::vector<float> min_distances(n, std::numeric_limits<float>::max());
    for (uint64_t c = 1; c < k; ++c) {
        const float* centroid = cent + (c - 1) * dim;
        for (uint64_t i = 0; i < n; ++i) {
            float dist = fp32_l2sqr(x + i * dim, centroid, dim);
            min_distances[i] = std::min(min_distances[i], dist);
        }
        double total_weight = 0.0;
        for (uint64_t i = 0; i < n; ++i) {
            total_weight += min_distances[i];
        }
        uint64_t selected = n - 1;
        if (total_weight <= 0.0) {
            double f = draws[c - 1] * static_cast<double>(n);
            selected = f >= static_cast<double>(n - 1) ? n - 1 : static_cast<uint64_t>(f);
        } else {
            double threshold = draws[c - 1] * total_weight;
            double cumulative = 0.0;
            for (uint64_t i = 0; i < n; ++i) {
                cumulative += min_distances[i];
                if (cumulative >= threshold) {
                    selected = i;
                    break;
                }
            }
        }
        picks[c] = selected;
        std::memcpy(cent + c * dim, x + selected * dim, dim * sizeof(float));
    }
}

// Lloyd driver (kmeans_cluster.cpp:46-190) with the initial centroids given and empty clusters
// re-seeded from mt19937(seed) + uniform_int_distribution<uint64_t>(0, n-1), drawn in cluster order.
// Returns the loss of the last assignment (err / n).  `assign` replaces the assignment step when given
// (a caller with a BLAS runs find_nearest_one_with_blas as the reference does, through SGEMM): it fills
// labels for the centroids it is handed and returns err / n.
typedef double (*orc_assign_fn)(const float* cent, int32_t* labels, void* user);

ORC_API double
orc_kmeans_run_with(const float* x, uint64_t n, uint64_t dim, float* cent /* in: init, out: final */, uint64_t k,
                    int iters, uint64_t seed, int32_t* labels, orc_assign_fn assign, void* user) {
    std::mt19937 gen(static_cast<uint32_t>(seed));
    std::vector<int32_t> counts(k);
    double err = 0;
    for (int it = 0; it < iters; ++it) {
        err = assign != nullptr ? assign(cent, labels, user) : orc_kmeans_assign(x, n, dim, cent, k, labels, nullptr);
        orc_kmeans_update(x, labels, n, dim, k, cent, counts.data());
        std::uniform_int_distribution<uint64_t> dis(0, n - 1);
        for (uint64_t j = 0; j < k; ++j) {
            if (counts[j] == 0) {
                uint64_t idx = dis(gen);
                std::memcpy(cent + j * dim, x + idx * dim, dim * sizeof(float));
            }
        }
    }
    return err;
}

ORC_API double
orc_kmeans_run(const float* x, uint64_t n, uint64_t dim, float* cent, uint64_t k, int iters, uint64_t seed,
               int32_t* labels) {
    return orc_kmeans_run_with(x, n, dim, cent, k, iters, seed, labels, nullptr, nullptr);
}

// ---- pqfs ------------------------------------------------------------------------------------
ORC_API void
orc_pq_encode(const float* x, uint64_t n, uint64_t dim, uint64_t pq_dim, const float* codebooks, int metric,
              uint8_t* codes) {
    const uint64_t cs = (pq_dim + 1) / 2;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(n); ++i) {
        pq_encode_one(x + i * dim, dim, pq_dim, codebooks, metric, codes + i * cs);
    }
}

// DecodeOneImpl (pq_fastscan_quantizer.cpp:140-156): the centroids the code names, subspace by subspace.
ORC_API void
orc_pq_decode(const uint8_t* codes, uint64_t n, uint64_t dim, uint64_t pq_dim, const float* codebooks, float* out) {
    const uint64_t cs = (pq_dim + 1) / 2, sd = dim / pq_dim;
    for (uint64_t r = 0; r < n; ++r) {
        for (uint64_t i = 0; i < pq_dim; ++i) {
            const float* c = codebooks + (i * kPqCentroids + pq_nibble(codes + r * cs, i)) * sd;
            std::memcpy(out + r * dim + i * sd, c, sd * sizeof(float));
        }
    }
}

ORC_API void
orc_pqfs_process_query(const float* q, uint64_t nq, uint64_t dim, uint64_t pq_dim, const float* codebooks, int metric,
                       uint8_t* out /* nq x (pq_dim * 16 + 8) */) {
    for (uint64_t i = 0; i < nq; ++i) {
        pqfs_process_query(q + i * dim, dim, pq_dim, codebooks, metric, out + i * (pq_dim * kPqCentroids + 8));
    }
}

ORC_API void
orc_pqfs_package32(const uint8_t* codes, uint64_t pq_dim, int64_t valid, uint8_t* packaged) {
    pqfs_package32(codes, pq_dim, valid, packaged);
}

ORC_API void
orc_pqfs_unpack32(const uint8_t* packaged, uint64_t pq_dim, uint8_t* codes) {
    pqfs_unpack32(packaged, pq_dim, codes);
}

ORC_API void
orc_pqfs_lookup32(const uint8_t* lut, const uint8_t* packaged, uint64_t pq_dim, int32_t* result) {
    pqfs_lookup32(lut, packaged, pq_dim, result);
}

// ScanBatchDistImpl (pq_fastscan_quantizer.cpp:166-199) over `count` codes packaged in blocks of 32 (the last
// block padded): dists[count].
ORC_API void
orc_pqfs_scan_batch(const uint8_t* q, const uint8_t* packaged, uint64_t count, uint64_t pq_dim, int metric,
                    float* dists) {
    const uint64_t cs = (pq_dim + 1) / 2;
    const float diff = rd_f32(q + pq_dim * kPqCentroids), lower = rd_f32(q + pq_dim * kPqCentroids + 4);
    for (uint64_t b = 0; b * 32 < count; ++b) {
        int32_t tmp[32] = {0};
        pqfs_lookup32(q, packaged + b * 32 * cs, pq_dim, tmp);
        for (uint64_t j = 0; j < 32 && b * 32 + j < count; ++j) {
            dists[b * 32 + j] = pqfs_map(tmp[j], diff, lower, metric);
        }
    }
}

// PQFastScanQuantizer::TrainImpl (pq_fastscan_quantizer.cpp:62-94): the first min(n, 65536) rows (normalised for
// cosine), sliced per subspace, 16 centroids by KMeansCluster::Run (k-means++ seeding, 25 Lloyd iterations).  The
// reference draws from std::random_device; here subspace i seeds mt19937(seed + i): `first` and the k-means++ draws
// come from it in that order, and the Lloyd run re-seeds empty clusters from mt19937(seed + i) as orc_kmeans_run does.
ORC_API void
orc_pq_train(const float* x, uint64_t n, uint64_t dim, uint64_t pq_dim, int metric, uint64_t seed, float* codebooks) {
    const uint64_t count = std::min<uint64_t>(n, 65536), sd = dim / pq_dim;
    std::vector<float> norm;
    const float* data = x;
    if (metric == kCosine) {
        norm.resize(count * dim);
        for (uint64_t i = 0; i < count; ++i) {
            normalize(x + i * dim, norm.data() + i * dim, dim);
        }
        data = norm.data();
    }
    std::vector<float> slice(count * sd);
    std::vector<int32_t> labels(count);
    for (uint64_t i = 0; i < pq_dim; ++i) {
        for (uint64_t j = 0; j < count; ++j) {
            std::memcpy(slice.data() + j * sd, data + j * dim + i * sd, sd * sizeof(float));
        }
        std::mt19937 gen(static_cast<uint32_t>(seed + i));
        std::uniform_int_distribution<uint64_t> first_dis(0, count - 1);
        const uint64_t first = first_dis(gen);
        std::uniform_real_distribution<double> unit(0.0, 1.0);
        std::vector<double> draws(kPqCentroids - 1);
        for (double& d : draws) {
            d = unit(gen);
            d = d < 1.0 ? d : 0.0;
        }
        float* cb = codebooks + i * kPqCentroids * sd;
        std::vector<uint64_t> picks(kPqCentroids);
        orc_kmeans_init_pp(slice.data(), count, sd, kPqCentroids, first, draws.data(), cb, picks.data());
        orc_kmeans_run(slice.data(), count, sd, cb, kPqCentroids, 25, seed + i, labels.data());
    }
}

// ---- flat scan with bounded heap (BruteForce::SearchWithRequest hot loop) ----------------------
// algorithm/bruteforce/bruteforce.cpp:518-551: every inner id in order, dist -> fixed-size max-heap;
// result packed ascending (inner_index_interface.cpp:1171-1200).  `queries` holds processed queries:
// fp32 rows for fp32/sq8/sq4, encoded query codes for the uniform kinds and RaBitQ.  Rows with fewer
// than k results are padded with id 0xFFFFFFFF / +inf.  OpenMP over queries mirrors the reference
// evaluator (tools/eval/case/search_eval_case.cpp:233-248).
ORC_API void
orc_flat_scan_topk(int kind, int metric, uint64_t dim, const uint8_t* codes, uint64_t n, uint64_t code_size,
                   const float* lb, const float* diff, int query_bits, const uint8_t* queries, uint64_t nq,
                   uint64_t query_stride, uint64_t k, int strict_heap, uint32_t* out_ids, float* out_dists,
                   int threads) {
    Store s{kind, metric, dim, code_size, codes, lb, diff, query_bits};
    RabitqLayout rl = rabitq_layout(dim, metric, query_bits ? query_bits : 4);
#ifdef _OPENMP
    if (threads > 0) {
        omp_set_num_threads(threads);
    }
#endif
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        const uint8_t* q = queries + qi * query_stride;
        uint32_t* ids = out_ids + qi * k;
        float* ds = out_dists + qi * k;
        uint64_t cnt;
        if (strict_heap) {
            StrictMaxHeap h(k);
            for (uint64_t i = 0; i < n; ++i) {
                h.push(store_dist(s, &rl, q, codes + i * code_size), static_cast<uint32_t>(i));
            }
            cnt = h.drain(ids, ds);
        } else {
            FixedMaxHeap h(k);
            for (uint64_t i = 0; i < n; ++i) {
                h.push(store_dist(s, &rl, q, codes + i * code_size), static_cast<uint32_t>(i));
            }
            cnt = h.drain(ids, ds);
        }
        for (uint64_t j = cnt; j < k; ++j) {
            ids[j] = 0xFFFFFFFFU;
            ds[j] = std::numeric_limits<float>::infinity();
        }
    }
}

// The same loop with the per-code distance supplied by the caller: used to time the reference's own
// compiled SIMD kernels (oracle/_ref, e.g. vsag::avx512::SQ8ComputeL2Sqr) under the BruteForce loop and
// heap restated above.  fn has the SQ8 / SQ4 signature (query, code, lower_bound, diff, dim); the value it
// returns is turned into a distance as scalar_quantizer.cpp:180-196 does (IP -> 1 - ip).
typedef float (*sq_dist_fn)(const float*, const uint8_t*, const float*, const float*, uint64_t);
ORC_API void
orc_flat_scan_topk_fn(void* fn_ptr, int metric, uint64_t dim, const uint8_t* codes, uint64_t n, uint64_t code_size,
                      const float* lb, const float* diff, const float* queries, uint64_t nq, uint64_t k,
                      uint32_t* out_ids, float* out_dists, int threads) {
    auto fn = reinterpret_cast<sq_dist_fn>(fn_ptr);
#ifdef _OPENMP
    if (threads > 0) {
        omp_set_num_threads(threads);
    }
#endif
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        const float* q = queries + qi * dim;
        FixedMaxHeap h(k);
        for (uint64_t i = 0; i < n; ++i) {
            float v = fn(q, codes + i * code_size, lb, diff, dim);
            h.push(metric == kL2 ? v : 1 - v, static_cast<uint32_t>(i));
        }
        uint64_t cnt = h.drain(out_ids + qi * k, out_dists + qi * k);
        for (uint64_t j = cnt; j < k; ++j) {
            out_ids[qi * k + j] = 0xFFFFFFFFU;
            out_dists[qi * k + j] = std::numeric_limits<float>::infinity();
        }
    }
}

// All (query, code) distances, for small parity cases.
ORC_API void
orc_flat_dists(int kind, int metric, uint64_t dim, const uint8_t* codes, uint64_t n, uint64_t code_size,
               const float* lb, const float* diff, int query_bits, const uint8_t* queries, uint64_t nq,
               uint64_t query_stride, float* out /* nq x n */) {
    Store s{kind, metric, dim, code_size, codes, lb, diff, query_bits};
    RabitqLayout rl = rabitq_layout(dim, metric, query_bits ? query_bits : 4);
#pragma omp parallel for schedule(static)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        for (uint64_t i = 0; i < n; ++i) {
            out[qi * n + i] = store_dist(s, &rl, queries + qi * query_stride, codes + i * code_size);
        }
    }
}

// ---- IVF --------------------------------------------------------------------------------------
// Exact routing: the nprobe nearest centroids by fp32 distance (the reference routes through an HGraph
// over the centroids, ivf_nearest_partition.cpp:99-147; its exact form is what `disable_bucket_scan`
// reports, ivf.cpp:1589-1660).  Ascending distance, ties by heap order.
ORC_API void
orc_ivf_route(const float* cent, uint64_t nlist, uint64_t dim, int metric, const float* queries, uint64_t nq,
              uint64_t nprobe, int32_t* out_buckets, float* out_dists) {
    Store s{kFP32, metric == kCosine ? kIP : metric, dim, dim * 4, reinterpret_cast<const uint8_t*>(cent), nullptr,
            nullptr, 0};
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        FixedMaxHeap h(nprobe);
        const auto* q = reinterpret_cast<const uint8_t*>(queries + qi * dim);
        for (uint64_t j = 0; j < nlist; ++j) {
            h.push(store_dist(s, nullptr, q, s.codes + j * s.code_size), static_cast<uint32_t>(j));
        }
        std::vector<uint32_t> ids(nprobe);
        std::vector<float> ds(nprobe);
        uint64_t cnt = h.drain(ids.data(), ds.data());
        for (uint64_t j = 0; j < nprobe; ++j) {
            out_buckets[qi * nprobe + j] = j < cnt ? static_cast<int32_t>(ids[j]) : -1;
            out_dists[qi * nprobe + j] = j < cnt ? ds[j] : std::numeric_limits<float>::infinity();
        }
    }
}

// Posting lists as the reference fills them without a thread pool (ivf.cpp:590-724,
// bucket_datacell.h:670-709): vectors appended to their bucket in input order -> a stable counting
// sort by label.  offsets has nlist+1 entries; order[p] is the inner id at posting position p.
ORC_API void
orc_ivf_build_lists(const int32_t* labels, uint64_t n, uint64_t nlist, uint64_t* offsets, uint32_t* order) {
    std::fill(offsets, offsets + nlist + 1, 0);
    for (uint64_t i = 0; i < n; ++i) {
        offsets[labels[i] + 1]++;
    }
    for (uint64_t j = 0; j < nlist; ++j) {
        offsets[j + 1] += offsets[j];
    }
    std::vector<uint64_t> cur(offsets, offsets + nlist);
    for (uint64_t i = 0; i < n; ++i) {
        order[cur[labels[i]]++] = static_cast<uint32_t>(i);
    }
}

// IVF::search<KNN> for one batch with routing injected (ivf.cpp:1693-1828): for each probed bucket in
// the given order, scan the list (bucket_datacell.h:527-572) and feed (dist, inner id) to one
// strict-`<` heap of size kcand (flat_bucket_searcher.cpp:62-104).  codes are in posting order.
ORC_API void
orc_ivf_scan(int kind, int metric, uint64_t dim, const uint8_t* codes, uint64_t code_size, const float* lb,
             const float* diff, int query_bits, const uint64_t* offsets, const uint32_t* order,
             const uint8_t* queries, uint64_t nq, uint64_t query_stride, const int32_t* buckets, uint64_t nprobe,
             uint64_t kcand, uint32_t* out_ids, float* out_dists, int threads) {
    Store s{kind, metric, dim, code_size, codes, lb, diff, query_bits};
    RabitqLayout rl = rabitq_layout(dim, metric, query_bits ? query_bits : 4);
#ifdef _OPENMP
    if (threads > 0) {
        omp_set_num_threads(threads);
    }
#endif
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        StrictMaxHeap h(kcand);
        const uint8_t* q = queries + qi * query_stride;
        for (uint64_t p = 0; p < nprobe; ++p) {
            int32_t b = buckets[qi * nprobe + p];
            if (b < 0) {
                continue;
            }
            for (uint64_t pos = offsets[b]; pos < offsets[b + 1]; ++pos) {
                h.push(store_dist(s, &rl, q, codes + pos * code_size), order[pos]);
            }
        }
        uint64_t cnt = h.drain(out_ids + qi * kcand, out_dists + qi * kcand);
        for (uint64_t j = cnt; j < kcand; ++j) {
            out_ids[qi * kcand + j] = 0xFFFFFFFFU;
            out_dists[qi * kcand + j] = std::numeric_limits<float>::infinity();
        }
    }
}

// ---- use_residual of BucketDataCell ------------------------------------------------------------------------
// Train / encode_vector (bucket_datacell.h:594-625): the quantizer sees x - c of the row's bucket, x normalised first
// for cosine.
ORC_API void
orc_residual_rows(const float* x, uint64_t n, uint64_t dim, int metric, const int32_t* labels, const float* cent,
                  float* out) {
    std::vector<float> tmp(dim);
    for (uint64_t i = 0; i < n; ++i) {
        const float* cur = x + i * dim;
        if (metric == kCosine) {
            normalize(cur, tmp.data(), dim);
            cur = tmp.data();
        }
        const float* c = cent + static_cast<uint64_t>(labels[i]) * dim;
        for (uint64_t d = 0; d < dim; ++d) {
            out[i * dim + d] = cur[d] - c[d];
        }
    }
}

// DecodeOneImpl of the uniform quantizers (sq4_uniform_quantizer.cpp:160-170, sq8_uniform_quantizer.cpp:140-145):
// double arithmetic, rounded to float on the store.
ORC_API void
orc_squ_decode(const uint8_t* codes, uint64_t n, uint64_t dim, int bits, int metric, float lb, float diff, float* data) {
    UniformLayout l = uniform_layout(dim, bits, metric);
    for (uint64_t i = 0; i < n; ++i) {
        const uint8_t* c = codes + i * l.code_size;
        for (uint64_t d = 0; d < dim; ++d) {
            if (bits == 4) {
                int v = (d & 1) != 0 ? (c[d >> 1] & 0xf0) >> 4 : (c[d >> 1] & 0x0f);
                data[i * dim + d] = v / 15.0 * diff + lb;
            } else {
                data[i * dim + d] = c[d] / 255.0 * diff + lb;
            }
        }
    }
}

// encode_vector, l2 (bucket_datacell.h:626-636): -2 <c, decoded> - <c, c>.
ORC_API void
orc_residual_bias(const float* decoded, uint64_t n, uint64_t dim, const int32_t* labels, const float* cent, float* bias) {
    for (uint64_t i = 0; i < n; ++i) {
        const float* c = cent + static_cast<uint64_t>(labels[i]) * dim;
        bias[i] = -2 * fp32_ip(c, decoded + i * dim, dim) - fp32_ip(c, c, dim);
    }
}

// IVF::search<KNN> over residual lists: ScanBucketById (bucket_datacell.h:527-572) takes the list's residual bias
// (l2) and <q, c> (twice for l2) off every distance; the computer's query is the raw query, normalised for cosine
// (FactoryComputer, :574-592).  `queries` holds the processed queries as in orc_ivf_scan, `raw_queries` the float
// rows the <q, c> terms are formed from, `bias` one value per posting position (null: zeros).
ORC_API void
orc_ivf_scan_residual(int kind, int metric, uint64_t dim, const uint8_t* codes, uint64_t code_size, const float* lb,
                      const float* diff, int query_bits, const uint64_t* offsets, const uint32_t* order,
                      const uint8_t* queries, uint64_t nq, uint64_t query_stride, const float* raw_queries,
                      const float* cent, const float* bias, const int32_t* buckets, uint64_t nprobe, uint64_t kcand,
                      uint32_t* out_ids, float* out_dists) {
    Store s{kind, metric, dim, code_size, codes, lb, diff, query_bits};
    RabitqLayout rl = rabitq_layout(dim, metric, query_bits ? query_bits : 4);
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        StrictMaxHeap h(kcand);
        const uint8_t* q = queries + qi * query_stride;
        std::vector<float> rq(dim);
        if (metric == kCosine) {
            normalize(raw_queries + qi * dim, rq.data(), dim);
        } else {
            std::memcpy(rq.data(), raw_queries + qi * dim, dim * sizeof(float));
        }
        for (uint64_t p = 0; p < nprobe; ++p) {
            int32_t b = buckets[qi * nprobe + p];
            if (b < 0) {
                continue;
            }
            float ip_distance = fp32_ip(rq.data(), cent + static_cast<uint64_t>(b) * dim, dim);
            if (metric == kL2) {
                ip_distance *= 2;
            }
            for (uint64_t pos = offsets[b]; pos < offsets[b + 1]; ++pos) {
                float d = store_dist(s, &rl, q, codes + pos * code_size);
                if (metric == kL2 && bias != nullptr) {
                    d = d - bias[pos];
                }
                d -= ip_distance;
                h.push(d, order[pos]);
            }
        }
        uint64_t cnt = h.drain(out_ids + qi * kcand, out_dists + qi * kcand);
        for (uint64_t j = cnt; j < kcand; ++j) {
            out_ids[qi * kcand + j] = 0xFFFFFFFFU;
            out_dists[qi * kcand + j] = std::numeric_limits<float>::infinity();
        }
    }
}

// FlattenReorder::Reorder (impl/reorder/flatten_reorder.cpp:52-114): exact fp32 distance of every
// candidate (in candidate order) into a strict-`<` heap of size k, packed ascending.
ORC_API void
orc_rerank_fp32(const float* raw, uint64_t dim, int metric, const float* queries, uint64_t nq, const uint32_t* cand,
                uint64_t kcand, uint64_t k, uint32_t* out_ids, float* out_dists) {
#pragma omp parallel for schedule(dynamic)
    for (int64_t qi = 0; qi < static_cast<int64_t>(nq); ++qi) {
        StrictMaxHeap h(k);
        const float* q = queries + qi * dim;
        for (uint64_t j = 0; j < kcand; ++j) {
            uint32_t id = cand[qi * kcand + j];
            if (id == 0xFFFFFFFFU) {
                continue;
            }
            const float* x = raw + static_cast<uint64_t>(id) * dim;
            float d = metric == kL2 ? fp32_l2sqr(q, x, dim) : 1 - fp32_ip(q, x, dim);
            h.push(d, id);
        }
        uint64_t cnt = h.drain(out_ids + qi * k, out_dists + qi * k);
        for (uint64_t j = cnt; j < k; ++j) {
            out_ids[qi * k + j] = 0xFFFFFFFFU;
            out_dists[qi * k + j] = std::numeric_limits<float>::infinity();
        }
    }
}

// 1 when the host CPU can run the reference's avx512 kernels (flags of src/simd/CMakeLists.txt:57).
ORC_API int
orc_cpu_has_avx512() {
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
           __builtin_cpu_supports("avx512dq") && __builtin_cpu_supports("avx512vl") &&
           __builtin_cpu_supports("avx512cd") && __builtin_cpu_supports("avx512ifma") &&
           __builtin_cpu_supports("avx512vbmi");
}
ORC_API int
orc_cpu_has_avx512vpopcntdq() {
    return __builtin_cpu_supports("avx512vpopcntdq");
}
ORC_API int
orc_cpu_has_avx2() {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
}

ORC_API int
orc_max_threads() {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
