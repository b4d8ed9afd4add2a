// Posting lists of sq4_uniform codes (and, l2 only, sq8_uniform codes; at most 128 dimensions) against large query
// batches, on the int8 matrix cores.
//
// The streaming IVF kernel (ivf.hip) is bound by vector-ALU issue: every (query, code) pair costs sixteen dot4
// instructions.  The distance of this quantizer is a function of integers only,
//
//      dist = fl((Nq + No - 2 <q, o>) * scalar_rate),      Nq, No the squared norms of the 4-bit codes,
//
// (distance.h, finish_distances; sq4_uniform_quantizer.cpp:168-223 of the reference), and v_mfma_i32_32x32x32_i8
// delivers <q, o> exactly.  "dist <= bound" is therefore the integer test 2 <q, o> - No >= Nq - tmax(bound), where
// tmax is the largest integer t with fl(t * scalar_rate) <= bound; the pairs that pass are exactly the ones the
// streaming kernel would admit under the same bound, and their distances are formed by the same three fp32
// operations.  Inner product and cosine, dist = 1 - (lb (sum_q + sum_o) + rate <q, o> + lb^2), have no integer form:
// there the test is float(<q, o>) >= A_q + g * sum_o with every rounding of the streaming formula (and of the test)
// charged against A_q, and what passes is re-checked with the streaming kernel's own operations.
// The kernel serves the probe columns behind the first one: the nearest list of every query has been
// scanned by the streaming kernel, which leaves the bound.
//
// sq8_uniform, l2 (sq8_uniform_quantizer.cpp:204-250): the same distance formula with byte values 0..255 on both
// sides; every integer in it stays below 2^24 up to 128 dimensions, so the test is an integer test again.  The
// matrix cores take signed bytes: code and query are both centred, o' = o - 128, q' = q - 128 (q' = 0 beyond the
// dimension), and with X = <q', o'> over the real dimensions
//      <q, o> = X + 128 sum_q + 128 sum_o - 128^2 dim.
// sum_o is kept per slot next to No (store.h, kMetaPayloadSum), sum_q is formed once per query.  The accumulator
// starts from C_o = ceil((256 sum_o - No) / 2), so the pipe delivers X + C_o, and 2 <q, o> - No >= Tq becomes
// X + C_o >= floor((Tq - 256 sum_q + 2 128^2 dim) / 2) -- a test that keeps every pair of the real one and at most
// the pairs one unit beyond it, which ivf_i8_finish_kernel drops when it forms the distance.  Inner product and
// cosine: the float test of the 4-bit codes on the centred product, float(X) >= A'_q + g' sum_o with
// A'_q = A_q - 128 sum_q + 128^2 dim and the per-code term g m_o - 128 sum_o (m_o the code's stored scalar, the sum of
// the vector's values; sum_o the sum of its code values as under l2).
//
// Work split: the (query, list) pairs are grouped by list as for the streaming kernel; a workgroup is a chunk of a
// list's tiles and up to 256 of its pairs, four waves of 64.  It walks the chunk two tiles per LDS stage; staging
// splits the nibbles, so a staged tile looks like eight 16-byte granules per code in the operand order of the
// instruction.  What passes goes into the private list of (pair, chunk, lane / 32): no atomics.  A list that
// overflows raises the query's gate; gated queries drop these lists and are served by the streaming kernel.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kIvfI8Pairs = 256;  // pairs per workgroup
constexpr int kIvfI8StageTiles = 2;
// Lists are cut into chunks of about kIvfI8ChunkTiles tiles, at most kIvfI8Chunks per list (longer lists get longer
// chunks), so that one long list does not outlast the rest of the grid.
constexpr uint32_t kIvfI8ChunkTiles = 32;
constexpr uint32_t kIvfI8Chunks = 4;

__host__ __device__ inline uint32_t
ivf_i8_list_chunks(uint32_t tiles) {
    const uint32_t chunks = (tiles + kIvfI8ChunkTiles - 1) / kIvfI8ChunkTiles;
    return chunks < kIvfI8Chunks ? chunks : kIvfI8Chunks;
}

// Per query: Tq = Nq - tmax(bound) (see the header), widened by one level; the slow path re-checks exactly.
__global__ void __launch_bounds__(256)
ivf_i8_threshold_kernel(const uint32_t* bound, const float* qmeta, uint32_t qmeta_stride, int is_l2, float lb, float rate,
                        float lb2, uint32_t dpad, uint32_t centred_dim, const uint32_t* qtab, uint32_t qstride, uint64_t nq,
                        int32_t* tq) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q > nq) {
        return;
    }
    // Inner product: tq holds the bits of the float A_q.
    const int32_t never = is_l2 ? 0x7FFFFFFF : 0x7F800000, always = static_cast<int32_t>(is_l2 ? 0x80000000U : 0xFF800000U);
    if (q == nq) {
        tq[q] = never;  // the all-zero query row idle lanes point at: nothing passes
        return;
    }
    const uint32_t b = bound[q];
    if (b == 0xFFFFFFFFU || !(rate > 0.0F)) {
        tq[q] = always;  // no bound: everything passes (and the query will overflow)
        return;
    }
    const float bd = ordered_to_float(b);
    if (!is_l2) {
        // out = fl(1 - fl(fl(fl(lb fl(qm + m0)) + fl(rate ip)) + lb2)) <= bd.  With the real r* = lb (qm + m0) +
        // rate ip + lb2: |r - r*| and the rounding of 1 - r stay below 8u of the magnitudes involved, so
        // out <= bd implies rate ip >= 1 - bd - lb2 - lb qm - lb m0 - eps.
        constexpr double kU = 5.9604644775390625e-8;
        const double qm = static_cast<double>(qmeta[q * qmeta_stride]);
        // centred_dim != 0: byte codes (values up to 255), the product centred by 128 on both sides.
        const double vmax = centred_dim != 0 ? 255.0 : 15.0;
        const double m0_max = vmax * dpad, ip_max = vmax * vmax * dpad;
        const double mag = fabs(static_cast<double>(lb)) * (fabs(qm) + m0_max) + static_cast<double>(rate) * ip_max +
                           fabs(static_cast<double>(lb2)) + 1.0 + fabs(static_cast<double>(bd));
        double aq = (1.0 - bd - lb2 - static_cast<double>(lb) * qm - 16.0 * kU * mag) / static_cast<double>(rate);
        double slope = fabs(static_cast<double>(lb) / rate);
        if (centred_dim != 0) {
            // <q, o> = X + 128 sum_q + 128 sum_o - 128^2 dim: the test is on X.
            uint32_t sum = 0;
            const uint32_t* row = qtab + q * qstride;
            for (uint32_t w = 0; 4 * w < centred_dim; ++w) {
                uint32_t v = row[w];
                if (4 * w + 4 > centred_dim) {
                    v &= 0xFFFFFFFFU >> (8 * (4 * w + 4 - centred_dim));
                }
                sum = __builtin_amdgcn_udot4(v, 0x01010101U, sum, false);
            }
            aq += -128.0 * sum + 16384.0 * centred_dim;
            slope += 128.0;
        }
        // the test adds fl(g m0) to A_q in fp32 (g itself rounded, for byte codes twice)
        aq -= 8.0 * kU * (fabs(aq) + slope * m0_max + ip_max);
        float f = static_cast<float>(aq);
        if (static_cast<double>(f) > aq) {
            f = nextafterf(f, -__builtin_inff());
        }
        tq[q] = __float_as_int(f);
        return;
    }
    const double t0 = floor(static_cast<double>(bd) / static_cast<double>(rate));
    int64_t t = t0 > 1.0e9 ? 1000000000LL : (t0 < -1.0e9 ? -1000000000LL : static_cast<int64_t>(t0));
    for (int i = 0; i < 4 && static_cast<float>(t + 1) * rate <= bd; ++i) {
        ++t;
    }
    for (int i = 0; i < 4 && static_cast<float>(t) * rate > bd; ++i) {
        --t;
    }
    const int64_t nqv = static_cast<int64_t>(qmeta[q * qmeta_stride]);
    int64_t v = nqv - (t + 1);
    v = v > 0x7FFFFFFELL ? 0x7FFFFFFELL : (v < -0x7FFFFFFFLL ? -0x7FFFFFFFLL : v);
    tq[q] = static_cast<int32_t>(v);
}

// sq8_uniform: sum_q per query from its byte row, and the threshold of the centred product (see the header) in place
// of Tq.  One thread per query; tq[nq] (the dummy row) and the two sentinels stay as they are.
__global__ void __launch_bounds__(256)
ivf_i8_centre_threshold_kernel(const uint32_t* qtab, uint32_t qstride, uint32_t dim, uint64_t nq, int is_l2, int32_t* tq,
                               int32_t* qsum) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q > nq) {
        return;
    }
    uint32_t sum = 0;
    if (q < nq) {
        const uint32_t* row = qtab + q * qstride;
        for (uint32_t w = 0; 4 * w < dim; ++w) {
            uint32_t v = row[w];
            if (4 * w + 4 > dim) {
                v &= 0xFFFFFFFFU >> (8 * (4 * w + 4 - dim));
            }
            sum = __builtin_amdgcn_udot4(v, 0x01010101U, sum, false);
        }
    }
    qsum[q] = static_cast<int32_t>(sum);
    if (!is_l2) {
        return;  // the float threshold is centred where it is formed
    }
    const int32_t t = tq[q];
    if (t == 0x7FFFFFFF || t == static_cast<int32_t>(0x80000000U)) {
        return;
    }
    int64_t v = (static_cast<int64_t>(t) - 256LL * sum + 32768LL * dim) >> 1;  // floor
    v = v > 0x7FFFFFFELL ? 0x7FFFFFFELL : (v < -0x7FFFFFFFLL ? -0x7FFFFFFFLL : v);
    tq[q] = static_cast<int32_t>(v);
}

struct IvfI8Args {
    const uint4* tiles;
    uint32_t G;                  // granules per code (sq4_uniform <= 4, sq8_uniform <= 8)
    uint32_t dim;
    const uint32_t* meta;        // per slot: No as float bits
    const uint32_t* meta_sum;    // sq8_uniform: per slot, the sum of the code values
    const uint32_t* ids;         // inner id per tile slot
    const uint32_t* list_tile;   // 2 nlist: first tile and end of the used tiles of every list
    const uint32_t* pair_off;    // nlist + 1
    const uint32_t* item_off;    // nlist + 1: workgroups per list (256 pairs each), prefix sums
    const uint32_t* sorted_pair; // pair index (q * nprobe + p) grouped by list
    uint32_t nlist, nprobe;
    uint32_t dummy_query;        // index of the all-zero query row
    const uint32_t* qtab;        // processed queries (distance.h): per code dword {low nibbles, high nibbles}
    uint32_t qstride;
    const float* qmeta;
    uint32_t qmeta_stride;
    float lb, rate, lb2;         // the quantizer's constants (distance.h: f0, f1, f2)
    const int32_t* tq;           // per query (+ the dummy row)
    const uint32_t* bound;       // per query, ordered distance
    uint32_t k;                  // capacity of a private list
    uint64_t* partial;           // [pair][chunk][lane / 32][k] keys
    uint32_t* partial_cnt;       // [pair][chunk][lane / 32]
    uint32_t* gate;              // per query: raised when one of its lists overflowed; gate[nq] counts them
};

struct IvfI8Stage {
    // sq4_uniform: [2 granule + nibble half][code], one nibble per byte; sq8_uniform: [granule][code], bytes - 128
    uint4 codes[kIvfI8StageTiles][8 * kWave];
    int32_t term[kIvfI8StageTiles][kWave];     // what the accumulator of a code starts from (-No; sq8_uniform: C_o)
};

// ceil((256 sum_o - No) / 2); 256 sum_o >= No because every value is at most 255.
__device__ inline int32_t
ivf_i8_centre_term(uint32_t sum_o, float no) {
    return (static_cast<int32_t>(256U * sum_o) - static_cast<int32_t>(no) + 1) >> 1;
}

template <int KIND, int METRIC>
__global__ void __launch_bounds__(256, 2)
ivf_i8_kernel(IvfI8Args p) {
    constexpr bool kBytes = KIND == VSAG_AMD_KIND_SQ8_UNIFORM;  // a byte per dimension
    __shared__ IvfI8Stage stage[2];
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
    // Which list: last b with item_off[b] <= item.
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
    // Items of a list: (block of 256 pairs) x (tile chunk), chunk fastest.
    const uint32_t list_begin = as_const(p.list_tile)[2 * b], list_end = as_const(p.list_tile)[2 * b + 1];
    const uint32_t chunks = ivf_i8_list_chunks(list_end - list_begin);
    const uint32_t per = chunks != 0 ? (list_end - list_begin + chunks - 1) / chunks : 0;
    const uint32_t chunk = chunks != 0 ? (item - ioff[b]) % chunks : 0;
    const uint32_t group = chunks != 0 ? (item - ioff[b]) / chunks : 0;
    uint32_t tile_begin = list_begin + chunk * per;
    tile_begin = tile_begin < list_end ? tile_begin : list_end;
    const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
    const uint32_t pbeg = as_const(p.pair_off)[b] + group * kIvfI8Pairs + wave * kWave;
    const uint32_t pend = as_const(p.pair_off)[b + 1];
    const bool active = pbeg < pend;
    const uint32_t span = tile_end - tile_begin;
    const uint32_t nstages = (span + kIvfI8StageTiles - 1) / kIvfI8StageTiles;
    if (nstages == 0) {
        return;  // an empty chunk: its lists keep their zero counts
    }

    // Query operands: block j = pairs pbeg + 32 j + lane % 32; step s = granule s, this lane's nibble half.
    intx4 qv[2][4];
    int32_t tq[2];
    uint32_t pair[2], qidx[2];
    uint32_t ncand[2] = {0, 0};
    uint64_t my_list[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t idx = pbeg + 32 * j + l32;
        const bool live = idx < pend;
        pair[j] = live ? as_const(p.sorted_pair)[idx] : 0xFFFFFFFFU;
        qidx[j] = live ? pair[j] / p.nprobe : p.dummy_query;
        const uint4* rowp = reinterpret_cast<const uint4*>(p.qtab + static_cast<uint64_t>(qidx[j]) * p.qstride);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if constexpr (kBytes) {
                // Step s, this half: dimensions 32 s + 16 half ... + 15, centred; zero beyond the dimension (and for
                // the dummy row, whose threshold nothing meets anyway).
                const uint32_t d0 = 32 * s + 16 * half;
                uint4 x = make_uint4(0, 0, 0, 0);
                if (2 * s + half < p.G) {
                    x = rowp[2 * s + half];
                }
                auto centre = [&](uint32_t w, uint32_t d) {
                    const uint32_t c = w ^ 0x80808080U;
                    return d + 4 <= p.dim ? c : (d >= p.dim ? 0U : c & (0xFFFFFFFFU >> (8 * (d + 4 - p.dim))));
                };
                qv[j][s] = intx4{static_cast<int>(centre(x.x, d0)), static_cast<int>(centre(x.y, d0 + 4)),
                                 static_cast<int>(centre(x.z, d0 + 8)), static_cast<int>(centre(x.w, d0 + 12))};
                continue;
            }
            uint4 x0 = make_uint4(0, 0, 0, 0), x1 = make_uint4(0, 0, 0, 0);
            if (static_cast<uint32_t>(s) < p.G) {
                x0 = rowp[2 * s];
                x1 = rowp[2 * s + 1];
            }
            qv[j][s] = half == 0 ? intx4{static_cast<int>(x0.x), static_cast<int>(x0.z), static_cast<int>(x1.x),
                                         static_cast<int>(x1.z)}
                                 : intx4{static_cast<int>(x0.y), static_cast<int>(x0.w), static_cast<int>(x1.y),
                                         static_cast<int>(x1.w)};
            if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                // Twice the query (0..30 still fits a signed byte): with the accumulator started from -No the matrix
                // pipe delivers 2 <q, o> - No, the quantity the test compares.
                qv[j][s] = qv[j][s] << 1;
            }
        }
        tq[j] = p.tq[qidx[j]];
        my_list[j] = (static_cast<uint64_t>(live ? pair[j] : 0) * kIvfI8Chunks + chunk) * 2 + half;
    }

    // Staging: wave w copies granule w of both tiles of the stage, a lane per code; the nibbles are split on the
    // way into LDS.  Wave t also brings the -No terms of tile t.
    // (sq8_uniform: wave w copies granules w and w + 4, centring the bytes.)
    uint4 regs[kIvfI8StageTiles][kBytes ? 2 : 1];
    int32_t my_term = 0;
    auto fetch = [&](uint32_t sg) {
#pragma unroll
        for (int tt = 0; tt < kIvfI8StageTiles; ++tt) {
            const uint32_t tile = tile_begin + sg * kIvfI8StageTiles + tt;
#pragma unroll
            for (int r = 0; r < (kBytes ? 2 : 1); ++r) {
                const uint32_t g = wave + 4 * r;
                const uint32_t none = kBytes ? 0x80808080U : 0U;
                regs[tt][r] = make_uint4(none, none, none, none);
                if (tile < tile_end && g < p.G) {
                    regs[tt][r] = p.tiles[(static_cast<uint64_t>(tile) * p.G + g) * kWave + lane];
                }
            }
            if (wave == static_cast<uint32_t>(tt)) {
                // l2: -No; inner product: the bits of g * sum_o, g = -lb / rate.  Padding tiles never pass.
                my_term = METRIC == VSAG_AMD_METRIC_L2 ? static_cast<int32_t>(0xC0000000U) : 0x7F800000;
                if (tile < tile_end) {
                    const float m0 = __uint_as_float(p.meta[static_cast<uint64_t>(tile) * kWave + lane]);
                    if constexpr (kBytes && METRIC == VSAG_AMD_METRIC_L2) {
                        my_term = ivf_i8_centre_term(p.meta_sum[static_cast<uint64_t>(tile) * kWave + lane], m0);
                    } else if constexpr (kBytes) {
                        const uint32_t so = p.meta_sum[static_cast<uint64_t>(tile) * kWave + lane];
                        my_term = __float_as_int(m0 * (-p.lb / p.rate) - 128.0F * static_cast<float>(so));
                    } else {
                        my_term = METRIC == VSAG_AMD_METRIC_L2 ? -static_cast<int32_t>(m0)
                                                               : __float_as_int(m0 * (-p.lb / p.rate));
                    }
                }
            }
        }
    };
    auto park = [&](IvfI8Stage& st) {
#pragma unroll
        for (int tt = 0; tt < kIvfI8StageTiles; ++tt) {
            if constexpr (kBytes) {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const uint4 v = regs[tt][r];
                    st.codes[tt][(wave + 4 * r) * kWave + lane] =
                        make_uint4(v.x ^ 0x80808080U, v.y ^ 0x80808080U, v.z ^ 0x80808080U, v.w ^ 0x80808080U);
                }
            } else {
                const uint4 v = regs[tt][0];
                st.codes[tt][(2 * wave) * kWave + lane] =
                    make_uint4(v.x & 0x0F0F0F0FU, v.y & 0x0F0F0F0FU, v.z & 0x0F0F0F0FU, v.w & 0x0F0F0F0FU);
                st.codes[tt][(2 * wave + 1) * kWave + lane] =
                    make_uint4((v.x >> 4) & 0x0F0F0F0FU, (v.y >> 4) & 0x0F0F0F0FU, (v.z >> 4) & 0x0F0F0F0FU,
                               (v.w >> 4) & 0x0F0F0F0FU);
            }
            if (wave == static_cast<uint32_t>(tt)) {
                st.term[tt][lane] = my_term;
            }
        }
    };

    constexpr int kBlocks = 4 * kIvfI8StageTiles;
    fetch(0);
    park(stage[0]);
    __syncthreads();
    uint32_t cur = 0;
    for (uint32_t sg = 0; sg < nstages; ++sg) {
        if (sg + 1 < nstages) {
            fetch(sg + 1);
        }
        if (active) {
            const IvfI8Stage& st = stage[cur];
            const uint64_t slot0 = (static_cast<uint64_t>(tile_begin) + sg * kIvfI8StageTiles) * kWave;
            intx16 acc[2];  // one being filled, one being judged
            intx4 av[2][4];
            int32_t tm[2][16];
            auto read_row = [&](int r) {
                const int tt = r >> 1, i = r & 1;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint4 c = st.codes[tt][(2 * s + half) * kWave + 32 * i + l32];
                    av[r & 1][s] = intx4{static_cast<int>(c.x), static_cast<int>(c.y), static_cast<int>(c.z),
                                         static_cast<int>(c.w)};
                }
                // Element e of a lane is code 32 i + 8 (e / 4) + 4 (lane / 32) + e % 4 of the tile.
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int4 v = *reinterpret_cast<const int4*>(&st.term[tt][32 * i + 8 * g + 4 * half]);
                    tm[r & 1][4 * g] = v.x;
                    tm[r & 1][4 * g + 1] = v.y;
                    tm[r & 1][4 * g + 2] = v.z;
                    tm[r & 1][4 * g + 3] = v.w;
                }
            };
            auto multiply = [&](int blk, intx16& c) {
                const int r = blk >> 1, j = blk & 1;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    c[e] = METRIC == VSAG_AMD_METRIC_L2 ? tm[r & 1][e] : 0;
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[r & 1][s], qv[j][s], c, 0, 0, 0);
                }
            };
            read_row(0);
            multiply(0, acc[0]);
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                const int r = blk >> 1, j = blk & 1;
                const bool reads = j == 0 && blk + 2 < kBlocks;
                if (reads) {
                    read_row(r + 1);
                }
                if (blk + 1 < kBlocks) {
                    multiply(blk + 1, acc[(blk + 1) & 1]);
                }
                // What passes is recorded as (slot, accumulator) and turned into (distance, id) by
                // ivf_i8_finish_kernel: nothing here waits for a load from global memory.
                auto record = [&](int e) {
                    const uint64_t slot = slot0 + 32 * r + 8 * (e >> 2) + 4 * half + (e & 3);
                    if (ncand[j] < p.k) {
                        p.partial[my_list[j] * p.k + ncand[j]] =
                            (slot << 32) | static_cast<uint32_t>(acc[blk & 1][e]);
                    }
                    ++ncand[j];
                };
                if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                    // Nearly nothing passes.  The sixteen elements of a lane are reduced to their best one with
                    // three-operand max instructions, four at a time, so that a block with a hit finds it group by
                    // group, and one compare decides whether the block needs a second look.
                    int32_t gbest[4];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        gbest[g] = max(max(max(acc[blk & 1][4 * g], acc[blk & 1][4 * g + 1]), acc[blk & 1][4 * g + 2]),
                                       acc[blk & 1][4 * g + 3]);
                    }
                    const bool hit = max(max(max(gbest[0], gbest[1]), gbest[2]), gbest[3]) >= tq[j];
                    const uint64_t any = __ballot(hit);
                    if (blk + 1 < kBlocks) {
                        if (reads) {
                            __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
                        }
#pragma unroll
                        for (int m = 0; m < 4; ++m) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                        }
                    }
                    if (any != 0) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            if (__ballot(gbest[g] >= tq[j]) == 0) {
                                continue;
                            }
#pragma unroll
                            for (int e = 4 * g; e < 4 * g + 4; ++e) {
                                const bool pass = acc[blk & 1][e] >= tq[j] && pair[j] != 0xFFFFFFFFU;
                                if (__ballot(pass) != 0 && pass) {
                                    record(e);
                                }
                            }
                        }
                    }
                } else {
                    // The sixteen verdicts stay in scalar registers; only a block with a hit builds a mask per lane.
                    bool pass[16];
                    uint64_t any = 0;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        pass[e] = static_cast<float>(acc[blk & 1][e]) >= __int_as_float(tm[r & 1][e]) + __int_as_float(tq[j]);
                        any |= __ballot(pass[e]);
                    }
                    if (blk + 1 < kBlocks) {
                        if (reads) {
                            __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
                        }
#pragma unroll
                        for (int m = 0; m < 4; ++m) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 12, 0);
                        }
                    }
                    if (any != 0) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            if (pass[e] && pair[j] != 0xFFFFFFFFU) {
                                record(e);
                            }
                        }
                    }
                }
            }
        }
        if (sg + 1 < nstages) {
            park(stage[cur ^ 1]);
        }
        __syncthreads();  // the next stage is complete, and every wave is done with this one
        cur ^= 1;
    }
    if (active) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (pair[j] != 0xFFFFFFFFU) {
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

// One thread per private list: its (slot, accumulator) records become (distance, id) keys through the streaming
// kernel's own three operations on the same integers; records of empty slots and of distances beyond the query's
// bound (the integer test is a level wider than the bound) are dropped and the list is closed up.
struct IvfI8FinishArgs {
    uint64_t* partial;
    uint32_t* partial_cnt;
    uint64_t lists;  // pairs x lists per pair
    uint32_t k, nprobe, p0, per_pair;  // probe columns p0 .. nprobe - 1 hold records, the ones before them keys
    const uint32_t* ids;
    const uint32_t* meta;
    const uint32_t* meta_sum;  // sq8_uniform: sum of the code values per slot
    const int32_t* qsum;       // sq8_uniform: sum of the query's values
    uint32_t dim;
    const float* qmeta;
    uint32_t qmeta_stride;
    const uint32_t* bound;
    float lb, rate, lb2;
};

template <int KIND, int METRIC>
__global__ void __launch_bounds__(256)
ivf_i8_finish_kernel(IvfI8FinishArgs p) {
    const uint64_t list = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (list >= p.lists) {
        return;
    }
    const uint64_t pair = list / p.per_pair;
    if (pair % p.nprobe < p.p0) {
        return;
    }
    const uint32_t count = p.partial_cnt[list];
    if (count == 0) {
        return;
    }
    const uint64_t q = pair / p.nprobe;
    const float qm = p.qmeta[q * p.qmeta_stride];
    const uint32_t bound = p.bound[q];
    uint64_t* keys = p.partial + list * p.k;
    // Four records at a time: their loads (record, then id and scalars of its slot) are in flight together, which is
    // what a full list -- a query with a loose bound -- waits for.  Kept keys go to the front of the list, never past
    // the records already read.
    uint32_t kept = 0;
    for (uint32_t i0 = 0; i0 < count; i0 += 4) {
        uint64_t recs[4];
        uint32_t idv[4];
        float m0v[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            recs[u] = keys[i0 + u < count ? i0 + u : count - 1];
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            idv[u] = p.ids[recs[u] >> 32];
            m0v[u] = __uint_as_float(p.meta[recs[u] >> 32]);
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint64_t slot = recs[u] >> 32;
            const int32_t acc = static_cast<int32_t>(static_cast<uint32_t>(recs[u]));
            const uint32_t id = idv[u];
            if (i0 + u >= count || id == VSAG_AMD_INVALID_ID) {
                continue;
            }
            const float m0 = m0v[u];
            float dist;
            if constexpr (KIND == VSAG_AMD_KIND_SQ8_UNIFORM && METRIC != VSAG_AMD_METRIC_L2) {
                // acc = X, <q, o> = X + 128 sum_q + 128 sum_o - 128^2 dim
                const int32_t ip = acc + 128 * p.qsum[q] + static_cast<int32_t>(128U * p.meta_sum[slot]) -
                                   static_cast<int32_t>(16384U * p.dim);
                const float result = static_cast<float>(ip);
                const float rr = p.lb * (qm + m0) + p.rate * result + p.lb2;
                dist = 1 - rr;
            } else if constexpr (KIND == VSAG_AMD_KIND_SQ8_UNIFORM) {
                // acc = X + C_o, <q, o> = X + 128 sum_q + 128 sum_o - 128^2 dim (see the header)
                const uint32_t so = p.meta_sum[slot];
                const int32_t ip = acc - ivf_i8_centre_term(so, m0) + 128 * p.qsum[q] + static_cast<int32_t>(128U * so) -
                                   static_cast<int32_t>(16384U * p.dim);
                const float result = static_cast<float>(ip);
                dist = (qm + m0 - 2 * result) * p.rate;
            } else if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
                // acc = 2 <q, o> - No with No = m0, an integer
                const float result = static_cast<float>((acc + static_cast<int32_t>(m0)) >> 1);
                dist = (qm + m0 - 2 * result) * p.rate;
            } else {
                const float result = static_cast<float>(acc);
                const float rr = p.lb * (qm + m0) + p.rate * result + p.lb2;
                dist = 1 - rr;
            }
            if (float_to_ordered(dist) <= bound) {
                keys[kept++] = make_key(dist, id);
            }
        }
    }
    p.partial_cnt[list] = kept;
}

// Gated queries: one of their private lists overflowed, so the streaming kernel scans lists again for them.  Which:
// the pairs (query, list) whose own private lists overflowed -- the other lists of the query are whole and stay -- as
// long as the direct launch has room for all such pairs (gpairs_cap); beyond that every pair of a gated query, through
// the streaming kernel's own grouping, and then nothing the matrix-core pass left for the query may count.  Two
// launches, a thread per pair: the first counts the overflowed pairs (gate[nq + 1]), the second empties the private lists
// of the pairs to scan again and queues them (gate[nq + 2] counts the queue; in the second case gate[nq + 1] is left
// above the capacity, which is what the streaming launches look at).
__device__ inline bool
ivf_pair_overflowed(const uint32_t* partial_cnt, uint64_t pair, uint32_t k) {
    bool over = false;
    for (uint32_t l = 0; l < 2 * kIvfI8Chunks; ++l) {
        over = over || partial_cnt[2 * kIvfI8Chunks * pair + l] > k;
    }
    return over;
}

__global__ void __launch_bounds__(256)
ivf_i8_count_gated_kernel(uint32_t* gate, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* partial_cnt,
                          const int32_t* buckets, uint32_t k) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint64_t per = nprobe - p0;
    if (i >= nq * per || gate[nq] == 0) {
        return;
    }
    const uint64_t q = i / per;
    if (gate[q] != 0) {
        const uint64_t pair = q * nprobe + p0 + i % per;
        if (buckets[pair] >= 0 && ivf_pair_overflowed(partial_cnt, pair, k)) {
            atomicAdd(&gate[nq + 1], 1U);
        }
    }
}

__global__ void __launch_bounds__(256)
ivf_i8_clear_gated_kernel(uint32_t* gate, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t* partial_cnt,
                          const int32_t* buckets, uint32_t* gpairs, uint32_t gpairs_cap, uint32_t k) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint64_t per = nprobe - p0;
    if (i >= nq * per || gate[nq] == 0) {
        return;
    }
    const uint64_t q = i / per;
    if (gate[q] != 0) {
        const uint64_t pair = q * nprobe + p0 + i % per;
        const bool by_pair = gate[nq + 1] <= gpairs_cap;  // fixed by the first launch
        if (by_pair && !ivf_pair_overflowed(partial_cnt, pair, k)) {
            return;
        }
        for (uint32_t l = 0; l < 2 * kIvfI8Chunks; ++l) {
            partial_cnt[2 * kIvfI8Chunks * pair + l] = 0;
        }
        if (by_pair && buckets[pair] >= 0) {
            gpairs[atomicAdd(&gate[nq + 2], 1U)] = static_cast<uint32_t>(pair);
        }
    }
}

// Private lists per (query, list) pair.
uint32_t
ivf_i8_lists_per_pair() {
    return 2 * kIvfI8Chunks;
}

bool
ivf_i8_supports(const vsag_amd_store* s) {
    if (s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
        return s->G <= 8 && s->dim <= 128 && s->nmeta == 2 && s->nlist > 0 && s->scalar_rate > 0.0F;
    }
    return s->kind == VSAG_AMD_KIND_SQ4_UNIFORM && s->G <= 4 && s->nlist > 0 && s->scalar_rate > 0.0F;
}

// After a matrix-core pass over probe columns [p0, nprobe): the private lists of the queries whose gate it raised are
// emptied and their pairs queued (see ivf_i8_clear_gated_kernel).
int
launch_ivf_clear_gated(uint32_t* gate, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t* partial_cnt,
                       const int32_t* buckets, uint32_t* gpairs, uint32_t gpairs_cap, uint32_t k, hipStream_t st) {
    const uint64_t pairs = nq * (nprobe - p0);
    hipLaunchKernelGGL(ivf_i8_count_gated_kernel, dim3(static_cast<uint32_t>(div_up(pairs, 256))), dim3(256), 0, st, gate,
                       nq, nprobe, p0, partial_cnt, buckets, k);
    hipLaunchKernelGGL(ivf_i8_clear_gated_kernel, dim3(static_cast<uint32_t>(div_up(pairs, 256))), dim3(256), 0, st, gate,
                       nq, nprobe, p0, partial_cnt, buckets, gpairs, gpairs_cap, k);
    VA_HIP(hipGetLastError());
    return 0;
}

// The pairs of probe columns [p0, nprobe) are grouped by list (pair_off, sorted_pair) and item_off counts
// workgroups per list (blocks of 256 pairs x tile chunks: offsets_kernel with T = 256, kIvfI8ChunkTiles,
// kIvfI8Chunks); `bound` holds what the first columns left.  tq: 2 (nq + 1) words; gate: nq + 2 words, zeroed.
int
launch_ivf_i8(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
              const uint32_t* pair_off, const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound,
              int32_t* tq, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const int32_t* buckets,
              uint32_t* gpairs, uint32_t gpairs_cap, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const bool bytes = s->kind == VSAG_AMD_KIND_SQ8_UNIFORM;
    int32_t* qsum = tq + nq + 1;
    hipLaunchKernelGGL(ivf_i8_threshold_kernel, dim3(static_cast<uint32_t>(div_up(nq + 1, 256))), dim3(256), 0, st, bound,
                       a.qmeta, a.qmeta_stride, l2 ? 1 : 0, a.f0, a.f1, a.f2, s->dpad, bytes ? s->dim : 0U, a.qtab, a.qstride, nq,
                       tq);
    if (bytes) {
        hipLaunchKernelGGL(ivf_i8_centre_threshold_kernel, dim3(static_cast<uint32_t>(div_up(nq + 1, 256))), dim3(256), 0,
                           st, a.qtab, a.qstride, s->dim, nq, l2 ? 1 : 0, tq, qsum);
    }
    IvfI8Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.dim = s->dim;
    p.meta = a.meta;
    p.meta_sum = bytes ? a.meta + a.meta_stride : nullptr;
    p.ids = s->ids_dev;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.dummy_query = static_cast<uint32_t>(nq);
    p.qtab = a.qtab;
    p.qstride = a.qstride;
    p.qmeta = a.qmeta;
    p.qmeta_stride = a.qmeta_stride;
    p.lb = a.f0;
    p.rate = a.f1;
    p.lb2 = a.f2;
    p.tq = tq;
    p.bound = bound;
    p.k = kcand;
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    // At most one partly filled block of pairs per probed list, each cut into at most kIvfI8Chunks items.
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kIvfI8Pairs)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfI8Chunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    if (bytes && l2) {
        hipLaunchKernelGGL((ivf_i8_kernel<VSAG_AMD_KIND_SQ8_UNIFORM, VSAG_AMD_METRIC_L2>), grid, dim3(256), 0, st, p);
    } else if (bytes) {
        hipLaunchKernelGGL((ivf_i8_kernel<VSAG_AMD_KIND_SQ8_UNIFORM, VSAG_AMD_METRIC_IP>), grid, dim3(256), 0, st, p);
    } else if (l2) {
        hipLaunchKernelGGL((ivf_i8_kernel<VSAG_AMD_KIND_SQ4_UNIFORM, VSAG_AMD_METRIC_L2>), grid, dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL((ivf_i8_kernel<VSAG_AMD_KIND_SQ4_UNIFORM, VSAG_AMD_METRIC_IP>), grid, dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    VA_TRY(launch_ivf_clear_gated(gate, nq, nprobe, p0, partial_cnt, buckets, gpairs, gpairs_cap, kcand, st));
    IvfI8FinishArgs f{};
    f.partial = partial;
    f.partial_cnt = partial_cnt;
    f.per_pair = ivf_i8_lists_per_pair();
    f.lists = nq * nprobe * f.per_pair;
    f.k = kcand;
    f.nprobe = nprobe;
    f.p0 = p0;
    f.ids = s->ids_dev;
    f.meta = a.meta;
    f.meta_sum = p.meta_sum;
    f.qsum = qsum;
    f.dim = s->dim;
    f.qmeta = a.qmeta;
    f.qmeta_stride = a.qmeta_stride;
    f.bound = bound;
    f.lb = a.f0;
    f.rate = a.f1;
    f.lb2 = a.f2;
    const dim3 fgrid(static_cast<uint32_t>(div_up(f.lists, 256)));
    if (bytes && l2) {
        hipLaunchKernelGGL((ivf_i8_finish_kernel<VSAG_AMD_KIND_SQ8_UNIFORM, VSAG_AMD_METRIC_L2>), fgrid, dim3(256), 0, st, f);
    } else if (bytes) {
        hipLaunchKernelGGL((ivf_i8_finish_kernel<VSAG_AMD_KIND_SQ8_UNIFORM, VSAG_AMD_METRIC_IP>), fgrid, dim3(256), 0, st, f);
    } else if (l2) {
        hipLaunchKernelGGL((ivf_i8_finish_kernel<VSAG_AMD_KIND_SQ4_UNIFORM, VSAG_AMD_METRIC_L2>), fgrid, dim3(256), 0, st, f);
    } else {
        hipLaunchKernelGGL((ivf_i8_finish_kernel<VSAG_AMD_KIND_SQ4_UNIFORM, VSAG_AMD_METRIC_IP>), fgrid, dim3(256), 0, st, f);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
