// Pre-selection for large query batches on a flat RaBitQ store (1-bit codes, 4-bit queries, L2 or inner product),
// on the matrix cores.
//
// The streaming kernel forms <code bits, 4-bit query> with sixteen and/popcount pairs per code dword and query; that
// is what bounds it.  The same integer is a contraction of 0/1 values with the values 0..15.  The matrix cores take
// 4-bit and 6-bit floats at twice the rate of bytes (v_mfma_scale_f32_32x32x64_f8f6f4): a code bit is the fp4 value 1.0
// or 0, and a query value v goes in as the fp6 (e2m3) value (v - m) / 2 with an integer m of the query's own, one of
// 0, +-0.5 .. +-7.5, all of which that format holds exactly; the fp32 sums of at most 1024 such products are exact, and
// the contraction comes out as (ip - m x (set bits of the code)) / 2, which moves the third factor below by m and halves
// all four.  m is the integer nearest to -u3: what is left of the third factor is at most a half, so the thresholds of
// neighbouring codes differ by little -- the group test below lives on that.  The estimator that turns ip into a
// distance (distance.h, finish_distances) is, for a given
// query and code, an affine function of that integer with a slope of known sign, so "distance <= bound" is
// "ip >= thr(query, code)" with
//
//      thr = A_c u1 + B_c u2 + S_c u3 + u4,
//      A_c = err / (2 norm), B_c = (norm^2 [- raw^2]) A_c, S_c = set bits            (per code)
//      u1 = K_q / (qn qm0), u2 = 1 / (qn qm0), u3 = -qm1 / qm0, u4 = (qm2 + qm3) / qm0  (per query; K_q holds the bound)
//
// evaluated in fp32 and lowered by 1 + 1e-4 thr (several orders above the rounding of either form; the product is
// never negative, so a negative threshold needs no margin).  The pairs that
// pass are rescored by rescore_kernel with the streaming arithmetic, so the result is the streaming scan's bit for bit.
// Codes the derivation does not cover (zero norm, non-positive error factor, zero raw norm) are candidates of every
// query.
//
// Work split: the 4-bit queries of a group of 128 are turned into fp6 once and stay in LDS (72 KB for 768
// dimensions) in the operand order of the instruction; a wave owns storage tiles (64 codes; their bits come from the
// store's copy in operand order, 128 dimensions at a time and one load ahead, and become fp4 with seven vector
// instructions per 32 dimensions) and meets all
// 128 queries of the group: 8 accumulators, 8 matrix instructions per step of 64 dimensions.  A workgroup is eight waves,
// two per SIMD, so that one wave's verdicts run under the other's matrix instructions; no barrier inside the loop.
// What passes goes into the private list of (query, wave of the grid, lane / 32).
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

typedef int intx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kRbQueries = 128;  // queries per workgroup; kRbMaxG granules per code: the query group has to fit the LDS
constexpr uint32_t kRbWaves = 8;      // waves per workgroup, two per SIMD: one multiplies while the other decides
constexpr uint32_t kRbThreads = kRbWaves * kWave;
constexpr uint32_t kRbWaveFloats = 3 * kWave + 4 * 8;  // LDS floats of a wave's per-code constants

// The fp6 (e2m3) pattern (sign | exponent (2) | mantissa (3)) of k / 2 for an integer k in [-15, 15].
__device__ inline uint32_t
rb_fp6_half(int k) {
    // 0, 0.5 (subnormal 0.100), 1, 1.5 | 2, 2.5, 3, 3.5 (steps of 1/4 from 010.000) | 4 .. 7.5 (steps of 1/2 from 011.000)
    const uint32_t a = static_cast<uint32_t>(k < 0 ? -k : k);
    const uint32_t mag = a < 4 ? 4 * a : (a < 8 ? 16 + 2 * (a - 4) : 24 + (a - 8));
    return mag | (k < 0 ? 32U : 0U);
}

// 4-bit queries as fp6: per query row and code dword w, the 32 values of dimensions 32 w ... less the query's offset
// (offset[q], an integer in [0, 15], rabitq_tau_kernel's u5) and halved, as 24 bytes, value t in bits 6 t .. 6 t + 5;
// the first 16 bytes go to qa[q ndw + w], the last 8 to qb[q ndw + w].  Padding rows are zero (the fp6 value 0).
__global__ void __launch_bounds__(256)
rabitq_query_f6_kernel(const uint32_t* qtab, uint32_t qstride, uint32_t ndw, uint64_t nq, uint64_t nq_pad,
                       const float* offset, uint4* qa, uint2* qb) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= nq_pad * ndw) {
        return;
    }
    const uint64_t q = i / ndw;
    const uint32_t w = static_cast<uint32_t>(i % ndw);
    uint32_t out[6] = {0, 0, 0, 0, 0, 0};
    if (q < nq) {
        const uint4 v = *reinterpret_cast<const uint4*>(qtab + q * qstride + 4 * w);
        const int m = static_cast<int>(offset[q]);
#pragma unroll
        for (uint32_t t = 0; t < 32; ++t) {
            const uint32_t val = ((v.x >> t) & 1U) | (((v.y >> t) & 1U) << 1) | (((v.z >> t) & 1U) << 2) |
                                 (((v.w >> t) & 1U) << 3);
            const uint64_t code = static_cast<uint64_t>(rb_fp6_half(static_cast<int>(val) - m)) << ((6 * t) % 32);
            out[(6 * t) / 32] |= static_cast<uint32_t>(code);
            if ((6 * t) % 32 > 26) {
                out[(6 * t) / 32 + 1] |= static_cast<uint32_t>(code >> 32);
            }
        }
    }
    qa[i] = make_uint4(out[0], out[1], out[2], out[3]);
    qb[i] = make_uint2(out[4], out[5]);
}

// Per query: u1..u4 of the header, halved, and the offset m as u5 (u[j * nq_pad + q]).  -inf in u4: everything passes;
// +inf: nothing does.
__global__ void __launch_bounds__(256)
rabitq_tau_kernel(const float* qmeta, uint32_t qmeta_stride, const uint32_t* bound, int is_l2, uint32_t dpad, uint64_t nq,
                  uint64_t nq_pad, float* u) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q >= nq_pad) {
        return;
    }
    float u1 = 0.0F, u2 = 0.0F, u3 = 0.0F, u4 = __builtin_inff(), u5 = 0.0F;
    if (q < nq) {
        const float* qm = qmeta + q * qmeta_stride;
        const uint32_t b = bound[q];
        const double qm0 = qm[0], qm1 = qm[1], qm23 = static_cast<double>(qm[2]) + static_cast<double>(qm[3]);
        const double qn = qm[4], qr = qm[5];
        u4 = -__builtin_inff();
        if (b != 0xFFFFFFFFU && qm0 > 0.0 && qn > 0.0 && qn < 1.0e30 && qm0 < 1.0e30) {
            const double bd = ordered_to_float(b);
            double kq;
            bool usable = true;
            if (is_l2) {
                kq = qn * qn - bd;
            } else {
                kq = qn * qn - qr * qr + 2.0 * (1.0 - bd);
                if (fabs(qr) < 1.0e-5) {
                    // every code is at distance 1
                    usable = false;
                    u4 = 1.0 <= bd ? -__builtin_inff() : __builtin_inff();
                }
            }
            if (usable) {
                const double inv = 1.0 / (qn * qm0);
                const double v1 = kq * inv, v3 = -qm1 / qm0, v4 = qm23 / qm0 - 1.0;
                // Factors so large that the fp32 threshold would lose its margin: everything passes instead.
                if (fabs(v1) <= 1.0e4 && inv <= 1.0e4 && fabs(v3) <= 64.0 && fabs(v4) <= 1.0e5) {
                    // The relative margin rides on the factors: a positive threshold comes out 1e-4 lower, a
                    // negative one is passed by every (non-negative) product anyway.
                    // Everything is halved with the contraction (exactly: a power of two).
                    const double lower = 1.0 - 1.0e-4;
                    u1 = static_cast<float>(0.5 * v1 * lower);
                    u2 = static_cast<float>(0.5 * inv * lower);
                    // Less the query's offset m: the contraction of the matrix cores is (ip - m x set bits) / 2.
                    const double m = fmin(15.0, fmax(0.0, rint(v3 * lower)));
                    u5 = static_cast<float>(m);
                    u3 = static_cast<float>(0.5 * (v3 * lower - m));
                    // The threshold is a chain of three fp32 fma over terms that may cancel: it is off by at most
                    // 3 x 2^-24 of the sum of their magnitudes, whatever it comes to itself.  2^-20 of the largest
                    // magnitudes any code can bring (A_c <= kRbMaxA, |B_c| <= kRbMaxB, set bits <= dpad) is taken off.
                    const double reach = kRbMaxA * fabs(v1) + kRbMaxB * inv + dpad * fabs(v3) + fabs(v4);
                    u4 = static_cast<float>(0.5 * (v4 * lower - 9.5367431640625e-7 * reach));
                }
            }
        }
    }
    u[q] = u1;
    u[nq_pad + q] = u2;
    u[2 * nq_pad + q] = u3;
    u[3 * nq_pad + q] = u4;
    u[4 * nq_pad + q] = u5;
}

struct PrefilterRbArgs {
    const uint4* f4tiles;    // the code bits in operand order (store.h)
    const float4* f4const;   // per slot: A_c, B_c, S_c of the header and the flags
    const float* f4group;    // per tile: 32 floats, the extremes of the constants over each group of sixteen codes
    uint32_t G;
    uint64_t tile_begin, tile_end;
    const uint4* qa;       // fp6 queries: [query][4 G code dwords] first 16 bytes of the 24 of a dword's 32 values
    const uint2* qb;       // and the last 8
    const float* u;        // [4][nq_pad]
    uint64_t nq, nq_pad;
    uint32_t* cand;        // [query][sub_lists][sub_cap]
    uint32_t* cand_cnt;    // [query][sub_lists]
    uint32_t sub_cap;
    uint32_t groups;       // grid x; the grid has groups * kRbWaves waves per query group
    // Posting lists (LISTS): a workgroup is a chunk of a list's tiles x up to 128 of the (query, list) pairs that probe
    // the list -- the work split of ivf_i8.hip with 128 pairs per item -- and its queries are gathered by pair.
    const uint32_t* list_tile;    // 2 nlist: first tile and end of the used tiles of every list
    const uint32_t* pair_off;     // nlist + 1
    const uint32_t* item_off;     // nlist + 1: workgroups per list, prefix sums
    const uint32_t* sorted_pair;  // pair index (q * nprobe + p) grouped by list
    uint32_t nlist, nprobe;
    uint32_t dummy_query;         // a padding row of the query tables: zero operands, a threshold nothing meets
    uint32_t k;                   // capacity of a private list
    uint64_t* partial;            // [pair][8][k]: tile slots; the waves of a pair's items share its eight lists
    uint32_t* partial_cnt;        // [pair][8]: appended so far, also beyond k
    uint32_t* gate;               // per query: raised when one of its lists overflowed; gate[dummy_query] counts them
};

// Lists are cut into chunks of about kIvfRbChunkTiles tiles, at most kIvfRbChunks per list (the private lists of a pair
// are laid out for four chunks, as in ivf_i8.hip).  Long chunks: a workgroup fills a compute unit alone (the registers
// of its eight waves), so what it does before its first tile -- finding its list, gathering its queries -- is not
// hidden behind another workgroup and has to be spread over many tiles.
constexpr uint32_t kIvfRbChunkTiles = 128;
constexpr uint32_t kIvfRbChunks = 4;

// The fp4 operand of 32 code bits in the store's operand order: register v = elements 8 v .. 8 v + 7, 1.0 = 0b0010.
__device__ inline intx8
rb_fp4(uint32_t w) {
    const uint32_t m = 0x22222222U;
    intx4 v = intx4{static_cast<int>((w << 1) & m), static_cast<int>(w & m), static_cast<int>((w >> 1) & m),
                    static_cast<int>((w >> 2) & m)};
    return __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1);
}

// Granules of code bits a wave keeps on their way from memory: a granule feeds sixteen matrix instructions, about a
// quarter of the time its load takes, and two waves on a SIMD do not hide the rest.  The depth divides the granules of a
// code, so that granule j of every tile sits in register set j % depth.
__host__ __device__ constexpr uint32_t
rb_ring(uint32_t granules) {
    return granules > 1 && granules % 2 == 0 ? 2 : 1;
}

// KG: the granules of a code (the store's G), a parameter so that the registers of the ring are fixed.
template <bool LISTS, uint32_t KG>
__global__ void __launch_bounds__(kRbThreads, 2)
prefilter_rb_kernel(PrefilterRbArgs p) {
    extern __shared__ uint4 rb_lds[];
    __shared__ uint32_t pair_q[LISTS ? kRbQueries : 1];     // LISTS: the query of each of the item's pairs
    __shared__ uint32_t pair_list[LISTS ? kRbQueries : 1];  // and the first of its private lists in this chunk
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    constexpr uint32_t kRing = rb_ring(KG);
    constexpr uint32_t kUnroll = KG <= 6 ? KG : kRing;  // seven and eight granules, all unrolled, run out of registers
    const uint32_t ndw = 4 * KG;  // code dwords: dword 2 s + h is what half h of the wave brings to step s
    uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * kRbQueries;
    uint4* qs = rb_lds;                                                  // [dword][128 queries]: 16 of its 24 bytes
    uint2* qt = reinterpret_cast<uint2*>(rb_lds + ndw * kRbQueries);     // [dword][128 queries]: the other 8
    float* cc = reinterpret_cast<float*>(qt + ndw * kRbQueries) + wave * kRbWaveFloats;  // [3][64] per wave
    float* cg = cc + 3 * kWave;  // then [4 groups of 16 codes][8]: the extremes of the three constants
    uint64_t tile_first = p.tile_begin, span = p.tile_end - p.tile_begin;
    uint64_t t_first = static_cast<uint64_t>(blockIdx.x) * kRbWaves + wave, t_step = static_cast<uint64_t>(p.groups) * kRbWaves;

    if constexpr (LISTS) {
        const uint32_t item = blockIdx.x;
        cu32_p ioff = as_const(p.item_off);
        if (item >= ioff[p.nlist]) {
            return;  // the whole workgroup
        }
        // Which list: last b with item_off[b] <= item; its items are (block of 128 pairs) x (tile chunk), chunk fastest.
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
        uint32_t chunks = (list_end - list_begin + kIvfRbChunkTiles - 1) / kIvfRbChunkTiles;
        chunks = chunks < kIvfRbChunks ? chunks : kIvfRbChunks;
        if (chunks == 0) {
            return;
        }
        const uint32_t per = (list_end - list_begin + chunks - 1) / chunks;
        const uint32_t chunk = (item - ioff[b]) % chunks;
        const uint32_t group = (item - ioff[b]) / chunks;
        uint32_t tile_begin = list_begin + chunk * per;
        tile_begin = tile_begin < list_end ? tile_begin : list_end;
        const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
        if (tile_end == tile_begin) {
            return;  // an empty chunk: its lists keep their zero counts
        }
        const uint32_t pbeg = as_const(p.pair_off)[b] + group * kRbQueries;
        const uint32_t pend = as_const(p.pair_off)[b + 1];
        if (tid < kRbQueries) {
            const uint32_t idx = pbeg + tid;
            const bool live = idx < pend;
            const uint32_t pair = live ? as_const(p.sorted_pair)[idx] : 0U;
            pair_q[tid] = live ? pair / p.nprobe : p.dummy_query;
            pair_list[tid] = live ? pair * kIvfRbChunks * 2 : 0xFFFFFFFFU;
        }
        __syncthreads();
        q0 = 0;
        tile_first = tile_begin;
        span = tile_end - tile_begin;
        t_first = wave;
        t_step = kRbWaves;
    }
    // The row of the query tables behind local query ql of the workgroup.
    auto query_row = [&](uint32_t ql) -> uint64_t {
        if constexpr (LISTS) {
            return pair_q[ql];
        } else {
            return q0 + ql;
        }
    };

    // The query group, once: chunk c of query q to qs[c][q].
    if constexpr (LISTS) {
        // A list item lives for a few tiles per wave only: the rows are fetched four loads at a time, so that the
        // gather takes a few memory round trips instead of one per 16 bytes.
        const uint32_t total = ndw * kRbQueries;
        for (uint32_t i0 = tid; i0 < total; i0 += 4 * blockDim.x) {
            uint4 v[4];
            uint2 t[4];
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t i = i0 + r * blockDim.x;
                const uint32_t ic = i < total ? i : total - 1;
                const uint64_t at = query_row(ic / ndw) * ndw + ic % ndw;
                v[r] = p.qa[at];
                t[r] = p.qb[at];
            }
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t i = i0 + r * blockDim.x;
                if (i < total) {
                    qs[(i % ndw) * kRbQueries + i / ndw] = v[r];
                    qt[(i % ndw) * kRbQueries + i / ndw] = t[r];
                }
            }
        }
    } else {
        for (uint32_t i = tid; i < ndw * kRbQueries; i += blockDim.x) {
            const uint32_t ql = i / ndw, c = i % ndw;
            const uint64_t at = query_row(ql) * ndw + c;
            qs[c * kRbQueries + ql] = p.qa[at];
            qt[c * kRbQueries + ql] = p.qb[at];
        }
    }
    // Candidates so far of this lane's four queries (flat stores): in LDS, the registers go to the accumulators.
    uint32_t* ncand = reinterpret_cast<uint32_t*>(cc - wave * kRbWaveFloats + kRbWaves * kRbWaveFloats) + tid;
    // So do the four factors of each of those queries: uq[(4 qb + j) kRbThreads] is u(j + 1).
    float* uq = reinterpret_cast<float*>(ncand + 4 * kRbThreads);
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        ncand[qb * kRbThreads] = 0;
    }
    // Which private list of query q is this lane's (flat stores).  Formed where it is needed -- rarely: the empty
    // statement keeps the compiler from forming it once, ahead of the loop, and holding it in registers the matrix
    // instructions want.
    auto list_of = [&](uint64_t q) -> uint64_t {
        uint32_t groups = p.groups;
        asm volatile("" : "+s"(groups));
        return q * (groups * 2 * kRbWaves) + (blockIdx.x * kRbWaves + wave) * 2 + half;
    };
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        const uint64_t q = query_row(32 * qb + l32);
        uq[(4 * qb + 0) * kRbThreads] = p.u[q];
        uq[(4 * qb + 1) * kRbThreads] = p.u[p.nq_pad + q];
        uq[(4 * qb + 2) * kRbThreads] = p.u[2 * p.nq_pad + q];
        uq[(4 * qb + 3) * kRbThreads] = p.u[3 * p.nq_pad + q];
    }
    __syncthreads();
    // LISTS: a pair has eight private lists (two per chunk in ivf_i8.hip's layout); here a hit goes to the one of
    // (wave % 4, lane / 32), so that the waves of an item -- and of the other chunks of a long list, which use the same
    // eight -- spread what passes over all of them: the estimator is noisy, and a pair may bring hundreds.
    auto append_shared = [&](uint32_t ql, uint64_t slot) {
        const uint32_t first = pair_list[ql];
        if (first != 0xFFFFFFFFU) {
            const uint64_t list = static_cast<uint64_t>(first) + 2 * (wave & 3U) + half;
            const uint32_t pos = atomicAdd(&p.partial_cnt[list], 1U);
            if (pos < p.k) {
                p.partial[list * p.k + pos] = slot;
            } else if (atomicExch(&p.gate[pair_q[ql]], 1U) == 0U) {
                atomicAdd(&p.gate[p.dummy_query], 1U);
            }
        }
    };

    // A tile's constants are asked for one tile ahead, its bits kRing granules ahead (across the end of a tile): with
    // two waves on a SIMD nothing else would hide their way from memory.
    float4 next_const = make_float4(0.0F, 0.0F, 0.0F, 0.0F);
    float next_group = 0.0F;
    uint4 ring[kRing];
#pragma unroll
    for (uint32_t j = 0; j < kRing; ++j) {
        ring[j] = make_uint4(0U, 0U, 0U, 0U);
    }
    if (t_first < span) {
        const uint64_t tile = tile_first + t_first;
        next_const = p.f4const[tile * kWave + lane];
        next_group = p.f4group[tile * 32 + l32];
#pragma unroll
        for (uint32_t j = 0; j < kRing; ++j) {
            ring[j] = p.f4tiles[(tile * KG + j) * kWave + lane];
        }
    }
    // The query operands of the first two pairs of matrix instructions of a tile.
    uint4 qb_a[2];
    uint2 qb_t[2];
#pragma unroll
    for (uint32_t j = 0; j < 2; ++j) {
        qb_a[j] = qs[half * kRbQueries + 32 * j + l32];
        qb_t[j] = qt[half * kRbQueries + 32 * j + l32];
    }
    for (uint64_t t = t_first; t < span; t += t_step) {
        const uint64_t tile = tile_first + t;
        // The bits of this lane's two codes (rows l32 and 32 + l32 of the tile) that its half of the wave brings to
        // the two steps of a granule.
        const uint4* code_rows = p.f4tiles + tile * KG * kWave + lane;
        // Per-code constants, a lane per code; the extremes of each group of sixteen, a lane of either half per value.
        const float4 mine = next_const;
        const float group_value = next_group;
        const uint64_t tile_after = t + t_step < span ? tile + t_step : tile;
        next_const = p.f4const[tile_after * kWave + lane];
        next_group = p.f4group[tile_after * 32 + l32];
        const uint4* rows_after = p.f4tiles + tile_after * KG * kWave + lane;
        const uint32_t flags = __float_as_uint(mine.w);
        wave_lds_fence();  // the previous tile's verdicts have read these
        cc[lane] = mine.x;
        cc[kWave + lane] = mine.y;
        cc[2 * kWave + lane] = mine.z;
        if (half == 0) {
            cg[l32] = group_value;
        }
        const uint64_t special_mask = __ballot((flags & 2U) != 0);
        const uint64_t code_mask = __ballot((flags & 1U) != 0);
        wave_lds_fence();

        uint32_t tile_hits[4] = {0, 0, 0, 0};
        // The first matrix instruction of an accumulator starts from zero.
        floatx16 acc[4][2];
        floatx16 zero;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            zero[e] = 0.0F;
        }
#pragma unroll kUnroll
        for (uint32_t g = 0; g < KG; ++g) {
            // p.G is KG: asked at run time, the question keeps every granule a block of its own.  In one block the
            // compiler gathers the matrix instructions by accumulator, which takes every query operand of the tile into
            // registers at once.
            if (g < p.G) {
                const uint4 bits = ring[g % kRing];
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const intx8 a0 = rb_fp4(m == 0 ? bits.x : bits.y);
                    const intx8 a1 = rb_fp4(m == 0 ? bits.z : bits.w);
#pragma unroll
                    for (int qb = 0; qb < 4; ++qb) {
                        // The query operand was asked for two pairs of matrix instructions ago; its registers go to the
                        // pair after the next (of the next step, granule or -- the queries being the same -- tile).
                        const uint32_t pair = 4 * m + qb;
                        const uint4 b = qb_a[pair % 2];
                        const uint2 t = qb_t[pair % 2];
                        // six of the eight operand registers hold fp6 values; the other two stay undefined
                        const intx4 b4 = intx4{static_cast<int>(b.x), static_cast<int>(b.y), static_cast<int>(b.z),
                                               static_cast<int>(b.w)};
                        const intx4 t4 = intx4{static_cast<int>(t.x), static_cast<int>(t.y), 0, 0};
                        const intx8 bv = __builtin_shufflevector(b4, t4, 0, 1, 2, 3, 4, 5, -1, -1);
                        // A: fp4 (4), B: fp6 e2m3 (2); both scales 2^0 (the e8m0 pattern 127)
                        const bool first = g == 0 && m == 0;
                        acc[qb][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a0, bv, first ? zero : acc[qb][0], 4, 2,
                                                                                      0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
                        acc[qb][1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a1, bv, first ? zero : acc[qb][1], 4, 2,
                                                                                      0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
                        const uint32_t pair_then = pair + 2;
                        const uint32_t g_then = pair_then < 8 ? g : (g + 1 < KG ? g + 1 : 0);
                        const uint32_t dw_then = 4 * g_then + 2 * ((pair_then % 8) / 4) + half;
                        qb_a[pair % 2] = qs[dw_then * kRbQueries + 32 * (pair_then % 4) + l32];
                        qb_t[pair % 2] = qt[dw_then * kRbQueries + 32 * (pair_then % 4) + l32];
                    }
                }
                // its register set goes to the granule kRing further on, of this tile or the next
                ring[g % kRing] = g + kRing < KG ? code_rows[(g + kRing) * kWave] : rows_after[(g + kRing - KG) * kWave];
            }
        }

        // Element e of a lane is code 32 i + 8 (e / 4) + 4 (lane / 32) + e % 4 of the tile against query l32 of block qb.
        // Four elements (one float4 of each per-code constant) at a time keeps the registers of two waves per SIMD.
        // First the sixteen of a lane at once: their largest sum against the smallest threshold any of them can have
        // (the fp32 chain of five and the rounded centres are off by less than 10 x 2^-24 of the magnitudes, inside the
        // 2^-20 taken off u4; u2 is never negative).  Only where a lane of the wave gets past that are the sixteen
        // looked at one by one.
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float4 ge = *reinterpret_cast<const float4*>(&cg[(2 * i + half) * 8]);
            const float ge_half_s = cg[(2 * i + half) * 8 + 4];
#pragma unroll
            for (int qb = 0; qb < 4; ++qb) {
                const float u1 = uq[(4 * qb) * kRbThreads], u2 = uq[(4 * qb + 1) * kRbThreads];
                const float u3 = uq[(4 * qb + 2) * kRbThreads], u4 = uq[(4 * qb + 3) * kRbThreads];
                const float least = fmaf(ge.x, u1, fmaf(-ge.y, fabsf(u1), fmaf(ge.z, u2, fmaf(ge.w, u3,
                                    fmaf(-ge_half_s, fabsf(u3), u4)))));
                const floatx16& r = acc[qb][i];
                float top = fmaxf(fmaxf(r[0], r[1]), r[2]);
                top = fmaxf(fmaxf(top, r[3]), r[4]);
                top = fmaxf(fmaxf(top, r[5]), r[6]);
                top = fmaxf(fmaxf(top, r[7]), r[8]);
                top = fmaxf(fmaxf(top, r[9]), r[10]);
                top = fmaxf(fmaxf(top, r[11]), r[12]);
                top = fmaxf(fmaxf(top, r[13]), r[14]);
                top = fmaxf(top, r[15]);
                if (__ballot(top >= least) == 0) {
                    continue;
                }
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    // the same test on the four of a quarter before their own thresholds are formed
                    const float top4 = fmaxf(fmaxf(fmaxf(r[4 * gq], r[4 * gq + 1]), r[4 * gq + 2]), r[4 * gq + 3]);
                    if (__ballot(top4 >= least) == 0) {
                        continue;
                    }
                    const uint32_t row = 32 * i + 8 * gq + 4 * half;
                    const float4 va = *reinterpret_cast<const float4*>(&cc[row]);
                    const float4 vb = *reinterpret_cast<const float4*>(&cc[kWave + row]);
                    const float4 vs = *reinterpret_cast<const float4*>(&cc[2 * kWave + row]);
                    const float ca[4] = {va.x, va.y, va.z, va.w};
                    const float cb[4] = {vb.x, vb.y, vb.z, vb.w};
                    const float cs[4] = {vs.x, vs.y, vs.z, vs.w};
                    bool pass[4];
                    uint64_t any = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float thr = fmaf(cs[j], u3, fmaf(cb[j], u2, fmaf(ca[j], u1, u4)));
                        pass[j] = acc[qb][i][4 * gq + j] >= thr;
                        any |= __ballot(pass[j]);
                    }
                    if (any != 0) {
                        uint32_t hits = 0;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            hits |= pass[j] ? 1U << j : 0U;
                        }
                        if constexpr (LISTS) {
                            // Bit 16 i + 4 gq + j of the tile's verdicts for this lane's pair of block qb; appended
                            // after the tile, one atomic per pair instead of one per hit.
                            tile_hits[qb] |= hits << (16 * i + 4 * gq);
                            continue;
                        }
                        const uint64_t q = q0 + 32 * qb + l32;
                        uint32_t* list = LISTS ? nullptr : p.cand + list_of(q < p.nq ? q : 0) * p.sub_cap;
                        while (hits != 0) {
                            const uint32_t j = static_cast<uint32_t>(__builtin_ctz(hits));
                            hits &= hits - 1;
                            const uint32_t code = row + j;
                            const uint64_t slot = tile * kWave + code;
                            if (((code_mask >> code) & 1ULL) != 0 && ((special_mask >> code) & 1ULL) == 0) {
                                if constexpr (LISTS) {
                                    append_shared(32 * qb + l32, slot);
                                } else {
                                    const uint32_t have = ncand[qb * kRbThreads];
                                    if (have < p.sub_cap) {
                                        list[have] = static_cast<uint32_t>(slot);
                                    }
                                    ncand[qb * kRbThreads] = have + 1;
                                }
                            }
                        }
                    }
                }
            }
        }
        if constexpr (LISTS) {
            // Room for all hits of a pair in one go: the four counts are asked for before the first answer is needed.
            uint32_t count[4], base[4];
            uint64_t list[4];
#pragma unroll
            for (int qb = 0; qb < 4; ++qb) {
                uint32_t mask = tile_hits[qb];
                // bit 16 i + 4 gq + j is code 32 i + 8 gq + 4 half + j
                uint32_t keep = 0;
                for (uint32_t m = mask; m != 0; m &= m - 1) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctz(m));
                    const uint32_t code = 32 * (bit >> 4) + 8 * ((bit >> 2) & 3U) + 4 * half + (bit & 3U);
                    if (((code_mask >> code) & 1ULL) != 0 && ((special_mask >> code) & 1ULL) == 0) {
                        keep |= 1U << bit;
                    }
                }
                const uint32_t first = pair_list[32 * qb + l32];
                keep = first != 0xFFFFFFFFU ? keep : 0U;
                tile_hits[qb] = keep;
                count[qb] = static_cast<uint32_t>(__builtin_popcount(keep));
                list[qb] = static_cast<uint64_t>(first) + 2 * (wave & 3U) + half;
                base[qb] = count[qb] != 0 ? atomicAdd(&p.partial_cnt[list[qb]], count[qb]) : 0U;
            }
#pragma unroll
            for (int qb = 0; qb < 4; ++qb) {
                uint32_t pos = base[qb];
                for (uint32_t m = tile_hits[qb]; m != 0; m &= m - 1) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctz(m));
                    const uint32_t code = 32 * (bit >> 4) + 8 * ((bit >> 2) & 3U) + 4 * half + (bit & 3U);
                    if (pos < p.k) {
                        p.partial[list[qb] * p.k + pos] = tile * kWave + code;
                    }
                    ++pos;
                }
                if (count[qb] != 0 && pos > p.k) {
                    if (atomicExch(&p.gate[pair_q[32 * qb + l32]], 1U) == 0U) {
                        atomicAdd(&p.gate[p.dummy_query], 1U);
                    }
                }
            }
        }
        // Codes outside the derivation: candidates of every query (lanes of the first half append them).
        if (special_mask != 0 && half == 0) {
            uint64_t rest = special_mask;
            while (rest != 0) {
                const uint32_t code = static_cast<uint32_t>(__builtin_ctzll(rest));
                rest &= rest - 1;
#pragma unroll
                for (int qb = 0; qb < 4; ++qb) {
                    if constexpr (LISTS) {
                        append_shared(32 * qb + l32, tile * kWave + code);
                        continue;
                    }
                    const uint64_t q = q0 + 32 * qb + l32;
                    if (q < p.nq) {
                        const uint32_t have = ncand[qb * kRbThreads];
                        if (have < p.sub_cap) {
                            p.cand[list_of(q) * p.sub_cap + have] = static_cast<uint32_t>(tile * kWave + code);
                        }
                        ncand[qb * kRbThreads] = have + 1;
                    }
                }
            }
        }
    }
    if constexpr (!LISTS) {
#pragma unroll
        for (int qb = 0; qb < 4; ++qb) {
            const uint64_t q = q0 + 32 * qb + l32;
            if (q < p.nq) {
                p.cand_cnt[list_of(q)] = ncand[qb * kRbThreads];
            }
        }
    }
}

template <bool LISTS, uint32_t KG>
static int
launch_rb_kernel_g(dim3 grid, size_t lds, hipStream_t st, const PrefilterRbArgs& p) {
    VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(prefilter_rb_kernel<LISTS, KG>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    hipLaunchKernelGGL((prefilter_rb_kernel<LISTS, KG>), grid, dim3(kRbThreads), lds, st, p);
    return 0;
}

template <bool LISTS>
static int
launch_rb_kernel(uint32_t granules, dim3 grid, size_t lds, hipStream_t st, const PrefilterRbArgs& p) {
    switch (granules) {
        case 1: return launch_rb_kernel_g<LISTS, 1>(grid, lds, st, p);
        case 2: return launch_rb_kernel_g<LISTS, 2>(grid, lds, st, p);
        case 3: return launch_rb_kernel_g<LISTS, 3>(grid, lds, st, p);
        case 4: return launch_rb_kernel_g<LISTS, 4>(grid, lds, st, p);
        case 5: return launch_rb_kernel_g<LISTS, 5>(grid, lds, st, p);
        case 6: return launch_rb_kernel_g<LISTS, 6>(grid, lds, st, p);
        case 7: return launch_rb_kernel_g<LISTS, 7>(grid, lds, st, p);
        case 8: return launch_rb_kernel_g<LISTS, 8>(grid, lds, st, p);
        default: break;
    }
    return fail(VSAG_AMD_INVALID_ARGUMENT, "the rabitq matrix-core pass takes codes of at most %u granules, got %u", kRbMaxG,
                granules);
}

bool
prefilter_rb_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4 && s->nlist == 0 && s->G <= kRbMaxG && s->f4tiles != nullptr &&
           (s->metric == VSAG_AMD_METRIC_L2 || s->metric == VSAG_AMD_METRIC_IP);
}

uint64_t
prefilter_rb_padded_queries(uint64_t nq) {
    return div_up(nq, static_cast<uint64_t>(kRbQueries)) * kRbQueries;
}

// Bytes of scratch: the byte-expanded queries and the four per-query factors.
size_t
prefilter_rb_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    const uint64_t nq_pad = prefilter_rb_padded_queries(nq);
    return static_cast<size_t>(nq_pad) * s->G * 128 + static_cast<size_t>(nq_pad) * 20 + 512;
}

// Private candidate lists per query for nq queries over `span` tiles.
uint32_t
prefilter_rb_sub_lists(uint64_t nq, uint64_t span) {
    const uint64_t qgroups = div_up(nq, static_cast<uint64_t>(kRbQueries));
    // One workgroup fits a compute unit (its query group fills the LDS) and all of them take equally long: three to
    // six rounds of them, whichever leaves the last round fullest.
    const uint64_t cus = static_cast<uint64_t>(device_cu_count());
    uint64_t groups = 1;
    double best = 0.0;
    for (uint64_t rounds = 3; rounds <= 6; ++rounds) {
        const uint64_t g = std::max<uint64_t>(1, cus * rounds / qgroups);
        const double fill = static_cast<double>(g * qgroups) / static_cast<double>(cus * div_up(g * qgroups, cus));
        if (fill > best + 1e-9) {
            best = fill;
            groups = g;
        }
    }
    groups = std::max<uint64_t>(1, std::min<uint64_t>(groups, div_up(span, static_cast<uint64_t>(kRbWaves))));
    return static_cast<uint32_t>(2 * kRbWaves * groups);
}

int
launch_prefilter_rb(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                    const uint32_t* bound, uint8_t* scratch, uint32_t* cand, uint32_t* cand_cnt, uint32_t sub_lists,
                    uint32_t sub_cap, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t nq_pad = prefilter_rb_padded_queries(nq);
    const uint32_t ndw = s->G * 4;
    uint4* qa = reinterpret_cast<uint4*>(scratch);
    uint2* qb = reinterpret_cast<uint2*>(scratch + static_cast<size_t>(nq_pad) * ndw * 16);
    float* u = reinterpret_cast<float*>(scratch + round_up(static_cast<size_t>(nq_pad) * ndw * 32, 256));
    hipLaunchKernelGGL(rabitq_tau_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad, 256))), dim3(256), 0, st, a.qmeta,
                       a.qmeta_stride, bound, l2 ? 1 : 0, s->G * 128, nq, nq_pad, u);
    hipLaunchKernelGGL(rabitq_query_f6_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad * ndw, 256))), dim3(256), 0, st,
                       a.qtab, a.qstride, ndw, nq, nq_pad, u + 4 * nq_pad, qa, qb);
    VA_HIP(hipGetLastError());
    PrefilterRbArgs p{};
    p.f4tiles = s->f4tiles;
    p.f4const = s->f4const;
    p.f4group = reinterpret_cast<const float*>(s->f4group);
    p.G = s->G;
    p.tile_begin = tile_begin;
    p.tile_end = tile_end;
    p.qa = qa;
    p.qb = qb;
    p.u = u;
    p.nq = nq;
    p.nq_pad = nq_pad;
    p.cand = cand;
    p.cand_cnt = cand_cnt;
    p.sub_cap = sub_cap;
    p.groups = sub_lists / (2 * kRbWaves);
    VA_CHECK_ARG(sub_lists == prefilter_rb_sub_lists(nq, tile_end - tile_begin), "candidate lists do not match the grid");
    const size_t lds = static_cast<size_t>(4 * s->G) * kRbQueries * 24 + kRbWaves * kRbWaveFloats * sizeof(float) +
                       (4 + 16) * kRbThreads * sizeof(uint32_t);
    dim3 grid(p.groups, static_cast<uint32_t>(nq_pad / kRbQueries));
    timing_begin(st);
    VA_TRY(launch_rb_kernel<false>(s->G, grid, lds, st, p));
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

// ---- posting lists ------------------------------------------------------------------------------------------------
bool
ivf_rb_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4 && s->nlist > 0 && s->G <= kRbMaxG && s->f4tiles != nullptr &&
           s->residual_centroids_dev == nullptr &&
           (s->metric == VSAG_AMD_METRIC_L2 || s->metric == VSAG_AMD_METRIC_IP);
}

// Pairs per work item of the list kernel (offsets_kernel's T) and the tiles of a chunk.
uint32_t
ivf_rb_pairs_per_item() {
    return kRbQueries;
}

uint32_t
ivf_rb_chunk_tiles() {
    return kIvfRbChunkTiles;
}

// Bytes of scratch for nq queries and one padding row.
size_t
ivf_rb_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    return prefilter_rb_scratch_bytes(s, nq + 1);
}

// The pairs of probe columns [p0, nprobe) grouped by list (pair_off, sorted_pair; item_off: offsets_kernel with
// T = 128, ivf_rb_chunk_tiles(), four chunks at most) against the bounds the nearest lists left: what may still matter is
// recorded as a tile slot in one of the pair's eight private lists of kcand records in `partial`, counted in
// partial_cnt (zero before; a count above kcand raised the query's gate).  gate: nq + 2 words as in ivf_i8.hip.
int
launch_ivf_rb(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
              const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, uint8_t* scratch,
              uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const uint64_t nq_pad = prefilter_rb_padded_queries(nq + 1);
    const uint32_t ndw = s->G * 4;
    uint4* qa = reinterpret_cast<uint4*>(scratch);
    uint2* qb = reinterpret_cast<uint2*>(scratch + static_cast<size_t>(nq_pad) * ndw * 16);
    float* u = reinterpret_cast<float*>(scratch + round_up(static_cast<size_t>(nq_pad) * ndw * 32, 256));
    hipLaunchKernelGGL(rabitq_tau_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad, 256))), dim3(256), 0, st, a.qmeta,
                       a.qmeta_stride, bound, l2 ? 1 : 0, s->G * 128, nq, nq_pad, u);
    hipLaunchKernelGGL(rabitq_query_f6_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad * ndw, 256))), dim3(256), 0, st,
                       a.qtab, a.qstride, ndw, nq, nq_pad, u + 4 * nq_pad, qa, qb);
    VA_HIP(hipGetLastError());
    PrefilterRbArgs p{};
    p.f4tiles = s->f4tiles;
    p.f4const = s->f4const;
    p.f4group = reinterpret_cast<const float*>(s->f4group);
    p.G = s->G;
    p.qa = qa;
    p.qb = qb;
    p.u = u;
    p.nq = nq;
    p.nq_pad = nq_pad;
    p.groups = 1;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.dummy_query = static_cast<uint32_t>(nq);
    p.k = kcand;
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    const size_t lds = static_cast<size_t>(4 * s->G) * kRbQueries * 24 + kRbWaves * kRbWaveFloats * sizeof(float) +
                       (4 + 16) * kRbThreads * sizeof(uint32_t);
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kRbQueries)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfRbChunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    VA_TRY(launch_rb_kernel<true>(s->G, grid, lds, st, p));
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
