// Pre-selection for large query batches on a flat RaBitQ store (1-bit codes, 4-bit queries, L2 or inner product),
// on the int8 matrix cores.
//
// The streaming kernel forms <code bits, 4-bit query> with sixteen and/popcount pairs per code dword and query; that
// is what bounds it.  The same integer is a contraction of 0/1 bytes with 0..15 bytes, exact on
// v_mfma_i32_32x32x32_i8.  The estimator that turns it into a distance (distance.h, finish_distances) is, for a given
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
// Work split: the 4-bit queries of a group of 128 are expanded to bytes once and stay in LDS (96 KB for 768
// dimensions) in the operand order of the instruction; a wave owns storage tiles (64 codes; their bits come a granule
// at a time, one granule ahead, and are expanded to 0/1 bytes with three vector instructions per nibble) and meets all
// 128 queries of the group: 8 accumulators, 8 matrix instructions per expanded step.  A workgroup is eight waves,
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

constexpr uint32_t kRbQueries = 128;  // queries per workgroup
constexpr uint32_t kRbMaxG = 8;       // granules per code (1024 dimensions): the query group has to fit the LDS
constexpr uint32_t kRbWaves = 8;      // waves per workgroup, two per SIMD: one multiplies while the other decides
constexpr uint32_t kRbThreads = kRbWaves * kWave;
// Largest per-code factors the fp32 threshold takes (A_c, |B_c|; codes beyond them are candidates of every query): the
// per-query slack below is sized for them.  B_c grows with the square of the data's scale (norm x error factor / 2).
constexpr float kRbMaxA = 64.0F;
constexpr float kRbMaxB = 4096.0F;

// 4-bit queries as bytes: row q holds, per code dword w, the 32 values of dimensions 32 w ... (dpad bytes per row).
__global__ void __launch_bounds__(256)
rabitq_query_bytes_kernel(const uint32_t* qtab, uint32_t qstride, uint32_t ndw, uint64_t nq, uint64_t nq_pad,
                          uint8_t* qbytes) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= nq_pad * ndw) {
        return;
    }
    const uint64_t q = i / ndw;
    const uint32_t w = static_cast<uint32_t>(i % ndw);
    uint32_t planes[4] = {0, 0, 0, 0};
    if (q < nq) {
        const uint4 v = *reinterpret_cast<const uint4*>(qtab + q * qstride + 4 * w);
        planes[0] = v.x;
        planes[1] = v.y;
        planes[2] = v.z;
        planes[3] = v.w;
    }
    uint32_t out[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        uint32_t word = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t t = 4 * b + k;
            const uint32_t val = ((planes[0] >> t) & 1U) | (((planes[1] >> t) & 1U) << 1) | (((planes[2] >> t) & 1U) << 2) |
                                 (((planes[3] >> t) & 1U) << 3);
            word |= val << (8 * k);
        }
        out[b] = word;
    }
    uint4* dst = reinterpret_cast<uint4*>(qbytes + (q * ndw + w) * 32);
    dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
    dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
}

// Per query: u1..u4 of the header (u[j * nq_pad + q]).  -inf in u4: everything passes; +inf: nothing does.
__global__ void __launch_bounds__(256)
rabitq_tau_kernel(const float* qmeta, uint32_t qmeta_stride, const uint32_t* bound, int is_l2, uint32_t dpad, uint64_t nq,
                  uint64_t nq_pad, float* u) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q >= nq_pad) {
        return;
    }
    float u1 = 0.0F, u2 = 0.0F, u3 = 0.0F, u4 = __builtin_inff();
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
                    const double lower = 1.0 - 1.0e-4;
                    u1 = static_cast<float>(v1 * lower);
                    u2 = static_cast<float>(inv * lower);
                    u3 = static_cast<float>(v3 * lower);
                    // The threshold is a chain of three fp32 fma over terms that may cancel: it is off by at most
                    // 3 x 2^-24 of the sum of their magnitudes, whatever it comes to itself.  2^-20 of the largest
                    // magnitudes any code can bring (A_c <= kRbMaxA, |B_c| <= kRbMaxB, set bits <= dpad) is taken off.
                    const double reach = kRbMaxA * fabs(v1) + kRbMaxB * inv + dpad * fabs(v3) + fabs(v4);
                    u4 = static_cast<float>(v4 * lower - 9.5367431640625e-7 * reach);
                }
            }
        }
    }
    u[q] = u1;
    u[nq_pad + q] = u2;
    u[2 * nq_pad + q] = u3;
    u[3 * nq_pad + q] = u4;
}

struct PrefilterRbArgs {
    const uint4* tiles;
    uint32_t G;
    uint64_t tile_begin, tile_end;
    uint64_t n;
    const uint32_t* meta;  // norm, error factor, set bits, raw norm: meta_stride words apart
    uint64_t meta_stride;
    const uint4* qbytes;   // [query][2 G * 4 chunks of 16 bytes]
    const float* u;        // [4][nq_pad]
    uint64_t nq, nq_pad;
    uint32_t* cand;        // [query][sub_lists][sub_cap]
    uint32_t* cand_cnt;    // [query][sub_lists]
    uint32_t sub_cap;
    uint32_t groups;       // grid x; the grid has groups * kRbWaves waves per query group
    // Posting lists (LISTS): a workgroup is a chunk of a list's tiles x up to 128 of the (query, list) pairs that probe
    // the list -- the work split of ivf_i8.hip with 128 pairs per item -- and its queries are gathered by pair.
    const uint32_t* ids;          // inner id per tile slot (slots without a code hold VSAG_AMD_INVALID_ID)
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

__device__ inline int
rb_spread(uint32_t nibble) {
    // bit j of the nibble into byte j
    return static_cast<int>((nibble * 0x00204081U) & 0x01010101U);
}

template <int METRIC, bool LISTS = false>
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
    const uint32_t nchunks = 8 * p.G;  // 16-byte chunks per query row: chunk 2 s + h of step s = code dword s
    uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * kRbQueries;
    uint4* qs = rb_lds;                                                           // [chunk][128 queries]
    float* cc = reinterpret_cast<float*>(rb_lds + nchunks * kRbQueries) + wave * 3 * kWave;  // [3][64] per wave
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
        const uint32_t total = nchunks * kRbQueries;
        for (uint32_t i0 = tid; i0 < total; i0 += 4 * blockDim.x) {
            uint4 v[4];
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t i = i0 + r * blockDim.x;
                const uint32_t ic = i < total ? i : total - 1;
                v[r] = p.qbytes[query_row(ic / nchunks) * nchunks + ic % nchunks];
            }
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t i = i0 + r * blockDim.x;
                if (i < total) {
                    qs[(i % nchunks) * kRbQueries + i / nchunks] = v[r];
                }
            }
        }
    } else {
        for (uint32_t i = tid; i < nchunks * kRbQueries; i += blockDim.x) {
            const uint32_t ql = i / nchunks, c = i % nchunks;
            qs[c * kRbQueries + ql] = p.qbytes[query_row(ql) * nchunks + c];
        }
    }
    float u1[4], u2[4], u3[4], u4[4];
    uint32_t ncand[4] = {0, 0, 0, 0};
    const uint32_t sub_lists = p.groups * 2 * kRbWaves;
    const uint32_t my_sub = (blockIdx.x * kRbWaves + wave) * 2 + half;
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        const uint64_t q = query_row(32 * qb + l32);
        u1[qb] = p.u[q];
        u2[qb] = p.u[p.nq_pad + q];
        u3[qb] = p.u[2 * p.nq_pad + q];
        u4[qb] = p.u[3 * p.nq_pad + q];
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

    for (uint64_t t = t_first; t < span; t += t_step) {
        const uint64_t tile = tile_first + t;
        // The bits of this lane's two codes (rows l32 and 32 + l32 of the tile), a granule at a time and one ahead.
        const uint4* code_rows = p.tiles + tile * p.G * kWave + l32;
        uint4 bits[2], ahead[2];
        bits[0] = code_rows[0];
        bits[1] = code_rows[32];
        // Per-code constants, a lane per code.
        const uint64_t my_slot = tile * kWave + lane;
        const float bn = __uint_as_float(p.meta[my_slot]);
        float berr = __uint_as_float(p.meta[p.meta_stride + my_slot]);
        const float bsum = __uint_as_float(p.meta[2 * p.meta_stride + my_slot]);
        const float braw = METRIC == VSAG_AMD_METRIC_L2 ? 0.0F : __uint_as_float(p.meta[3 * p.meta_stride + my_slot]);
        if (fabsf(berr) < 1e-5F) {
            berr = berr >= 0 ? 1.0F : -1.0F;
        }
        // Outside the derivation, or with factors so large that the fp32 threshold would lose its margin.
        bool odd = !(bn > 0.0F) || !(berr > 0.0F) || !(bn < 1.0e18F) || !(berr < 1.0e18F);
        if (METRIC != VSAG_AMD_METRIC_L2) {
            odd = odd || !(fabsf(braw) >= 1e-5F) || !(fabsf(braw) < 1.0e18F);
        }
        float a_c = odd ? 0.0F : berr / (2.0F * bn);
        float b_c = odd ? 0.0F : (bn * bn - braw * braw) * a_c;
        odd = odd || !(a_c <= kRbMaxA) || !(fabsf(b_c) <= kRbMaxB) || !(fabsf(bsum) <= static_cast<float>(128 * p.G));
        a_c = odd ? 0.0F : a_c;
        b_c = odd ? 0.0F : b_c;
        bool holds_code = my_slot < p.n;
        if constexpr (LISTS) {
            holds_code = as_const(p.ids)[my_slot] != VSAG_AMD_INVALID_ID;
        }
        const bool special = odd && holds_code;
        wave_lds_fence();  // the previous tile's verdicts have read these
        cc[lane] = a_c;
        cc[kWave + lane] = b_c;
        cc[2 * kWave + lane] = odd ? 0.0F : bsum;
        const uint64_t special_mask = __ballot(special);
        const uint64_t code_mask = __ballot(holds_code);
        wave_lds_fence();

        uint32_t tile_hits[4] = {0, 0, 0, 0};
        intx16 acc[4][2];
#pragma unroll
        for (int qb = 0; qb < 4; ++qb) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[qb][i][e] = 0;
                }
            }
        }
#pragma unroll
        for (uint32_t g = 0; g < kRbMaxG; ++g) {
            if (g < p.G) {
                if (g + 1 < p.G) {
                    ahead[0] = code_rows[(g + 1) * kWave];
                    ahead[1] = code_rows[(g + 1) * kWave + 32];
                }
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const uint32_t s = 4 * g + m;
                    intx4 av[2];
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const uint32_t dw = m == 0 ? bits[i].x : (m == 1 ? bits[i].y : (m == 2 ? bits[i].z : bits[i].w));
                        const uint32_t hb = dw >> (16 * half);
                        av[i] = intx4{rb_spread(hb & 15U), rb_spread((hb >> 4) & 15U), rb_spread((hb >> 8) & 15U),
                                      rb_spread((hb >> 12) & 15U)};
                    }
#pragma unroll
                    for (int qb = 0; qb < 4; ++qb) {
                        const uint4 b = qs[(2 * s + half) * kRbQueries + 32 * qb + l32];
                        const intx4 bv = intx4{static_cast<int>(b.x), static_cast<int>(b.y), static_cast<int>(b.z),
                                               static_cast<int>(b.w)};
                        acc[qb][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[0], bv, acc[qb][0], 0, 0, 0);
                        acc[qb][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[1], bv, acc[qb][1], 0, 0, 0);
                    }
                }
                bits[0] = ahead[0];
                bits[1] = ahead[1];
            }
        }

        // Element e of a lane is code 32 i + 8 (e / 4) + 4 (lane / 32) + e % 4 of the tile against query l32 of block qb.
        // Four elements (one float4 of each per-code constant) at a time keeps the registers of two waves per SIMD.
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const uint32_t row = 32 * i + 8 * gq + 4 * half;
                const float4 va = *reinterpret_cast<const float4*>(&cc[row]);
                const float4 vb = *reinterpret_cast<const float4*>(&cc[kWave + row]);
                const float4 vs = *reinterpret_cast<const float4*>(&cc[2 * kWave + row]);
                const float ca[4] = {va.x, va.y, va.z, va.w};
                const float cb[4] = {vb.x, vb.y, vb.z, vb.w};
                const float cs[4] = {vs.x, vs.y, vs.z, vs.w};
#pragma unroll
                for (int qb = 0; qb < 4; ++qb) {
                    bool pass[4];
                    uint64_t any = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float thr = fmaf(cs[j], u3[qb], fmaf(cb[j], u2[qb], fmaf(ca[j], u1[qb], u4[qb])));
                        pass[j] = static_cast<float>(acc[qb][i][4 * gq + j]) >= thr;
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
                        uint32_t* list = LISTS ? nullptr : p.cand + ((q < p.nq ? q : 0) * sub_lists + my_sub) * p.sub_cap;
                        while (hits != 0) {
                            const uint32_t j = static_cast<uint32_t>(__builtin_ctz(hits));
                            hits &= hits - 1;
                            const uint32_t code = row + j;
                            const uint64_t slot = tile * kWave + code;
                            if (((code_mask >> code) & 1ULL) != 0 && ((special_mask >> code) & 1ULL) == 0) {
                                if constexpr (LISTS) {
                                    append_shared(32 * qb + l32, slot);
                                } else {
                                    if (ncand[qb] < p.sub_cap) {
                                        list[ncand[qb]] = static_cast<uint32_t>(slot);
                                    }
                                    ++ncand[qb];
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
                        if (ncand[qb] < p.sub_cap) {
                            p.cand[(q * sub_lists + my_sub) * p.sub_cap + ncand[qb]] = static_cast<uint32_t>(tile * kWave + code);
                        }
                        ++ncand[qb];
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
                p.cand_cnt[q * sub_lists + my_sub] = ncand[qb];
            }
        }
    }
}

bool
prefilter_rb_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4 && s->nlist == 0 && s->G <= kRbMaxG &&
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
    return static_cast<size_t>(nq_pad) * s->G * 128 + static_cast<size_t>(nq_pad) * 16 + 512;
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
    uint8_t* qbytes = scratch;
    float* u = reinterpret_cast<float*>(scratch + round_up(static_cast<size_t>(nq_pad) * ndw * 32, 256));
    hipLaunchKernelGGL(rabitq_query_bytes_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad * ndw, 256))), dim3(256), 0, st,
                       a.qtab, a.qstride, ndw, nq, nq_pad, qbytes);
    hipLaunchKernelGGL(rabitq_tau_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad, 256))), dim3(256), 0, st, a.qmeta,
                       a.qmeta_stride, bound, l2 ? 1 : 0, s->G * 128, nq, nq_pad, u);
    VA_HIP(hipGetLastError());
    PrefilterRbArgs p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.tile_begin = tile_begin;
    p.tile_end = tile_end;
    p.n = s->n;
    p.meta = a.meta;
    p.meta_stride = a.meta_stride;
    p.qbytes = reinterpret_cast<const uint4*>(qbytes);
    p.u = u;
    p.nq = nq;
    p.nq_pad = nq_pad;
    p.cand = cand;
    p.cand_cnt = cand_cnt;
    p.sub_cap = sub_cap;
    p.groups = sub_lists / (2 * kRbWaves);
    VA_CHECK_ARG(sub_lists == prefilter_rb_sub_lists(nq, tile_end - tile_begin), "candidate lists do not match the grid");
    const size_t lds = static_cast<size_t>(8 * s->G) * kRbQueries * 16 + kRbWaves * 3 * kWave * sizeof(float);
    dim3 grid(p.groups, static_cast<uint32_t>(nq_pad / kRbQueries));
    timing_begin(st);
    if (l2) {
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(prefilter_rb_kernel<VSAG_AMD_METRIC_L2>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        hipLaunchKernelGGL(prefilter_rb_kernel<VSAG_AMD_METRIC_L2>, grid, dim3(kRbThreads), lds, st, p);
    } else {
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(prefilter_rb_kernel<VSAG_AMD_METRIC_IP>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        hipLaunchKernelGGL(prefilter_rb_kernel<VSAG_AMD_METRIC_IP>, grid, dim3(kRbThreads), lds, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

// ---- posting lists ------------------------------------------------------------------------------------------------
bool
ivf_rb_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4 && s->nlist > 0 && s->G <= kRbMaxG &&
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
    uint8_t* qbytes = scratch;
    float* u = reinterpret_cast<float*>(scratch + round_up(static_cast<size_t>(nq_pad) * ndw * 32, 256));
    hipLaunchKernelGGL(rabitq_query_bytes_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad * ndw, 256))), dim3(256), 0, st,
                       a.qtab, a.qstride, ndw, nq, nq_pad, qbytes);
    hipLaunchKernelGGL(rabitq_tau_kernel, dim3(static_cast<uint32_t>(div_up(nq_pad, 256))), dim3(256), 0, st, a.qmeta,
                       a.qmeta_stride, bound, l2 ? 1 : 0, s->G * 128, nq, nq_pad, u);
    VA_HIP(hipGetLastError());
    PrefilterRbArgs p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.n = s->n;
    p.meta = a.meta;
    p.meta_stride = a.meta_stride;
    p.qbytes = reinterpret_cast<const uint4*>(qbytes);
    p.u = u;
    p.nq = nq;
    p.nq_pad = nq_pad;
    p.groups = 1;
    p.ids = s->ids_dev;
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
    const size_t lds = static_cast<size_t>(8 * s->G) * kRbQueries * 16 + kRbWaves * 3 * kWave * sizeof(float);
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kRbQueries)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfRbChunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    if (l2) {
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(prefilter_rb_kernel<VSAG_AMD_METRIC_L2, true>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        hipLaunchKernelGGL((prefilter_rb_kernel<VSAG_AMD_METRIC_L2, true>), grid, dim3(kRbThreads), lds, st, p);
    } else {
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(prefilter_rb_kernel<VSAG_AMD_METRIC_IP, true>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        hipLaunchKernelGGL((prefilter_rb_kernel<VSAG_AMD_METRIC_IP, true>), grid, dim3(kRbThreads), lds, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
