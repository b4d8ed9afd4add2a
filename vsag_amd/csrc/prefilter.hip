// Large query batches against a flat fp32 / sq8 store: the scan becomes a contraction on the matrix cores.
//
// With thousands of queries the streaming scan (scan.hip) is bound by vector-ALU issue, not by memory: every
// (query, code) pair costs d multiply-adds on the VALU.  The same inner products are an (N x d) * (d x nq)
// matrix product, which v_mfma_f32_32x32x2_f32 delivers several times faster -- but a product in the form
// |a|^2 - 2<a, y> + |y|^2 does not reproduce the reference's sum of (a_d - y_d)^2 bit for bit, and cancels badly
// for near-duplicates.  So the matrix product only pre-selects:
//
//   1. the streaming kernel scans a prefix of the store exactly; its k-th distance is a bound per query;
//   2. prefilter_kernel forms all inner products of the remaining codes with all queries tile by tile and
//      keeps the (query, code) pairs whose distance, minus a rigorous bound of the rounding error of the
//      product form, does not exceed the query's bound -- a few hundred candidates per query;
//   3. rescore_kernel recomputes these candidates with the streaming kernel's own arithmetic (the same
//      accumulate_granule in the same order) and selects from them as the streaming kernel would.
//
// The result is therefore the streaming result, bit for bit.  A query whose candidates overflow their buffer
// (no bound yet, masses of equal distances) is flagged and served by the streaming kernel over the remaining
// tiles instead.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PM = 128;  // codes per tile (two storage tiles)
constexpr int PN = 128;  // queries per tile
constexpr int PK = 32;   // contraction depth per stage
// Rows of a (parity, chunk) plane are PM float4; four more pad the plane so that the four chunks of one row
// start sixteen banks apart: a loader wave writes whole float4 slots of four rows x four chunks (or of 64
// consecutive rows of one chunk) without a bank conflict, and the MFMA lanes read 64 consecutive rows.
constexpr int kPfPlane = PM + 4;

// LDS operand layout of one stage: [parity h = k & 1][chunk c = k / 8][row] of float4, element e of the float4
// is k = 8 c + 2 e + h, so that a lane of the MFMA (row = lane % 32, h = lane / 32) reads its operand for four
// consecutive k-steps with one ds_read_b128.
struct PfStage {
    float4 a[2 * 4 * kPfPlane];
    float4 b[2 * 4 * kPfPlane];
};

// Eight consecutive k (k = 8c .. 8c+7 of `row`, lo = the first four) as the two float4 slots of chunk c.
__device__ inline void
pf_stage_store8(float4* plane, uint32_t row, uint32_t c, float4 lo, float4 hi) {
    plane[(0 * 4 + c) * kPfPlane + row] = make_float4(lo.x, lo.z, hi.x, hi.z);
    plane[(1 * 4 + c) * kPfPlane + row] = make_float4(lo.y, lo.w, hi.y, hi.w);
}

struct PrefilterArgs {
    const uint4* tiles;
    uint32_t G;
    uint64_t tile_begin, tile_end;  // storage tiles covered
    uint64_t n;                     // codes in the store (slots at or beyond are padding)
    const float* scale;             // sq8, l2: y_d = c_d * scale_d; null: y_d = c_d
    const float* qtab;              // processed queries, qstride floats per row, zero beyond the dimension
    uint32_t qstride;
    uint64_t nq;
    uint32_t kdim;                  // contraction length
    const float* term;              // per slot |y|^2
    float term_factor;              // 1 (l2) or 0 (ip)
    float dot_factor;               // -2 (l2) or -1 (ip)
    const float* tau;               // per query: keep a pair when term_factor |y|^2 + dot_factor <a, y> <= tau
    uint32_t* cand;                 // nq x cap slots
    uint32_t* cand_cnt;             // nq
    uint32_t cap;
    uint32_t groups;                // grid x; code tile t is walked by group t % groups
};

__device__ inline float4
pf_query_chunk(const float* qtab, uint64_t row, uint64_t rows, uint32_t k0, uint32_t stride) {
    if (row < rows && k0 + 4 <= stride) {
        return *reinterpret_cast<const float4*>(qtab + row * stride + k0);
    }
    return make_float4(0.0F, 0.0F, 0.0F, 0.0F);
}

template <int KIND>
__global__ void __launch_bounds__(256, 3)
prefilter_kernel(PrefilterArgs p) {
    // One 32 KiB stage: three workgroups (twelve waves, as many as the 170 registers of a wave allow) per compute
    // unit fill each other's barriers and loader phases, which pays more than double buffering with fewer waves.
    __shared__ PfStage stage[1];
    __shared__ float code_term[PM];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;   // which 64 codes of the tile
    const uint32_t wn = wave >> 1;  // which 64 queries of the tile
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * PN;
    const uint32_t ktiles = (p.kdim + PK - 1) / PK;
    const uint64_t span = p.tile_end - p.tile_begin;
    const uint64_t mtiles = (span + 1) / 2;

    // Query loader roles: 512 (row, chunk) pairs of eight floats per stage, two per thread; four lanes cover the
    // 128 contiguous bytes of a row.
    uint32_t qrow[2], qc[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        uint32_t idx = tid + 256 * r;
        qrow[r] = idx >> 2;
        qc[r] = idx & 3;
    }
    float tau_n[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint64_t q = q0 + wn * 64 + j * 32 + l32;
        tau_n[j] = q < p.nq ? p.tau[q] : -__builtin_inff();
    }

    // Code loader: a thread fetches granules of code `crow` of the tile (storage tile crow / 64, lane crow % 64).
    const uint32_t crow = tid & 127;
    const uint32_t cpart = tid >> 7;  // 0 / 1
    auto code_granule = [&](uint64_t mt, uint32_t j) {
        uint64_t tile = p.tile_begin + 2 * mt + (crow >> 6);
        if (tile < p.tile_end && j < p.G) {
            return p.tiles[(tile * p.G + j) * kWave + (crow & 63)];
        }
        return make_uint4(0, 0, 0, 0);
    };
    // sq8: a stage is 32 dimensions = granules 2 kt and 2 kt + 1, one per thread (chunks 2 cpart, 2 cpart + 1).
    // fp32: a stage is 32 dimensions = granules 8 kt .. 8 kt + 7; a thread takes chunks cpart and cpart + 2, two
    // granules each.
    constexpr int kCodeRegs = KIND == VSAG_AMD_KIND_SQ8 ? 1 : 4;
    auto fetch_codes = [&](uint64_t mt, uint32_t kt, uint4 (&regs)[kCodeRegs]) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
            regs[0] = code_granule(mt, 2 * kt + cpart);
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                regs[2 * r] = code_granule(mt, 8 * kt + 2 * (cpart + 2 * r));
                regs[2 * r + 1] = code_granule(mt, 8 * kt + 2 * (cpart + 2 * r) + 1);
            }
        }
    };
    auto as_floats = [](uint4 v) {
        return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    };
    auto park_codes = [&](float4* plane, uint32_t kt, const uint4 (&regs)[kCodeRegs]) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
            const uint32_t w[4] = {regs[0].x, regs[0].y, regs[0].z, regs[0].w};
            const uint32_t d0 = PK * kt + 16 * cpart;
            float4 v[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                v[m] = make_float4(static_cast<float>(w[m] & 0xffU), static_cast<float>((w[m] >> 8) & 0xffU),
                                   static_cast<float>((w[m] >> 16) & 0xffU), static_cast<float>(w[m] >> 24));
                if (p.scale != nullptr && d0 + 16 <= p.kdim) {
                    float4 sc = *reinterpret_cast<const float4*>(p.scale + d0 + 4 * m);
                    v[m].x *= sc.x;
                    v[m].y *= sc.y;
                    v[m].z *= sc.z;
                    v[m].w *= sc.w;
                }
            }
            pf_stage_store8(plane, crow, 2 * cpart, v[0], v[1]);
            pf_stage_store8(plane, crow, 2 * cpart + 1, v[2], v[3]);
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                pf_stage_store8(plane, crow, cpart + 2 * r, as_floats(regs[2 * r]), as_floats(regs[2 * r + 1]));
            }
        }
    };

    // Operands of stage 0 of the first tile; from then on the next tile's stage 0 is fetched while the last
    // stage of the current tile is multiplied, so that no tile starts by waiting for memory.
    uint4 rc[kCodeRegs];
    float4 rq[4];
    auto fetch_queries = [&](uint32_t kt) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            rq[2 * r] = pf_query_chunk(p.qtab, q0 + qrow[r], p.nq, PK * kt + 8 * qc[r], p.qstride);
            rq[2 * r + 1] = pf_query_chunk(p.qtab, q0 + qrow[r], p.nq, PK * kt + 8 * qc[r] + 4, p.qstride);
        }
    };
    auto park_queries = [&](float4* plane) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            pf_stage_store8(plane, qrow[r], qc[r], rq[2 * r], rq[2 * r + 1]);
        }
    };
    auto fetch_stage0 = [&](uint64_t mt) {
        fetch_codes(mt, 0, rc);
        fetch_queries(0);
    };
    if (blockIdx.x < mtiles) {
        fetch_stage0(blockIdx.x);
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
        // The stage is free: the previous tile's contraction ended with a barrier.
        park_codes(stage[0].a, 0, rc);
        park_queries(stage[0].b);
        float my_term = 0.0F;  // parked in LDS late: slower waves may still be reading the previous tile's terms
        if (tid < PM) {
            uint64_t slot = slot0 + tid;
            bool real = slot < p.n && p.tile_begin + 2 * mt + (tid >> 6) < p.tile_end;
            my_term = real ? p.term_factor * p.term[slot] : __builtin_inff();
        }
        __syncthreads();
        for (uint32_t kt = 0; kt < ktiles; ++kt) {
            if (kt + 1 < ktiles) {
                fetch_codes(mt, kt + 1, rc);
                fetch_queries(kt + 1);
            } else if (mt + p.groups < mtiles) {
                fetch_stage0(mt + p.groups);
            }
            const float4* pa = stage[0].a + half * 4 * kPfPlane + wm * 64 + l32;
            const float4* pb = stage[0].b + half * 4 * kPfPlane + wn * 64 + l32;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float4 a0 = pa[c * kPfPlane];
                float4 a1 = pa[c * kPfPlane + 32];
                float4 b0 = pb[c * kPfPlane];
                float4 b1 = pb[c * kPfPlane + 32];
                const float av0[4] = {a0.x, a0.y, a0.z, a0.w};
                const float av1[4] = {a1.x, a1.y, a1.z, a1.w};
                const float bv0[4] = {b0.x, b0.y, b0.z, b0.w};
                const float bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv0[e], acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv1[e], acc[0][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv0[e], acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv1[e], acc[1][1], 0, 0, 0);
                }
            }
            if (kt + 1 == ktiles && tid < PM) {
                // Every wave is past this tile's first barrier, hence out of the previous tile's epilogue.
                code_term[tid] = my_term;
            }
            __syncthreads();  // every wave has read the stage
            if (kt + 1 < ktiles) {
                park_codes(stage[0].a, kt + 1, rc);
                park_queries(stage[0].b);
                __syncthreads();
            }
        }
        // Nearly nothing passes: first collect the verdicts of all 64 products of this lane branch-free, then
        // let the rare lanes with a hit append.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t hits = 0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const float v = code_term[ml] + p.dot_factor * acc[i][j][e];
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
                    uint32_t pos = atomicAdd(&p.cand_cnt[q], 1U);
                    if (pos < p.cap) {
                        p.cand[q * p.cap + pos] = static_cast<uint32_t>(slot0 + ml);
                    }
                }
            }
        }
    }
}

// |y|^2 of the codes in slots [first, first + count) and the running maximum of |y| (as float bits; norms are
// not negative, so the bits order like the values).  One lane per code, dimensions in order.
template <int KIND>
__global__ void __launch_bounds__(256)
code_term_kernel(const uint4* tiles, uint32_t G, const float* scale, uint64_t first, uint64_t count, float* term,
                 uint32_t* ymax_bits) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    // Summed in double and rounded once: the int8 prefilter budgets two fp32 roundoffs for this term.
    double s = 0.0;
    if (i < count) {
        uint64_t slot = first + i;
        uint64_t tile = slot >> 6;
        uint32_t ln = static_cast<uint32_t>(slot & 63);
        for (uint32_t j = 0; j < G; ++j) {
            uint4 c = tiles[(tile * G + j) * kWave + ln];
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
            if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    double y = static_cast<double>((w[e >> 2] >> (8 * (e & 3))) & 0xffU);
                    if (scale != nullptr) {
                        y *= static_cast<double>(scale[16 * j + e]);
                    }
                    s = fma(y, y, s);
                }
            } else if constexpr (KIND == VSAG_AMD_KIND_SQ4) {
                // byte b of the granule: dimension 32 j + 2 b in its low nibble, 32 j + 2 b + 1 in its high one
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    double y = static_cast<double>((w[e >> 3] >> (8 * ((e >> 1) & 3) + 4 * (e & 1))) & 0xfU);
                    if (scale != nullptr) {
                        y *= static_cast<double>(scale[32 * j + e]);
                    }
                    s = fma(y, y, s);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    double y = static_cast<double>(__uint_as_float(w[e]));
                    s = fma(y, y, s);
                }
            }
        }
        term[slot] = static_cast<float>(s);
    }
    // A code with a NaN or infinite norm (fp32 stores hold whatever the caller gave) must not decide the maximum: it
    // would hide the largest finite norm, which the thresholds of all the other codes are built on.  Such a code's own
    // distances are NaN or infinite and order behind every finite one.
    float m = static_cast<float>(sqrt(s)) * (1.0F + 2.0e-7F);
    m = m < __builtin_inff() ? m : 0.0F;
    for (int off = 32; off > 0; off >>= 1) {
        m = fmaxf(m, __shfl_xor(m, off));
    }
    if ((threadIdx.x & 63) == 0 && m > 0.0F) {
        atomicMax(ymax_bits, __float_as_uint(m));
    }
}

// Per query: the admission threshold of the prefilter.  With dist = C_q + B <a, y> + F |y|^2 (l2: C = |a|^2,
// B = -2, F = 1; ip: C = 1 - qmeta, B = -1, F = 0) and the fp32 contraction of kdim terms off by at most
// kdim * 2^-22 * |a| * |y| (twice the worst case of sequential fp32 accumulation), a pair can only belong to the
// result when B <a, y> + F |y|^2 <= bound - C + |B| * err, plus the rounding of these few terms themselves.
__global__ void __launch_bounds__(64)
prefilter_tau_kernel(const float* qtab, uint32_t qstride, uint32_t kdim, const float* qmeta, uint32_t qmeta_stride,
                     int is_l2, const uint32_t* bound, const uint32_t* ymax_bits, uint64_t nq, float* tau,
                     float* magnitude_out = nullptr) {
    uint64_t q = blockIdx.x;
    uint32_t lane = threadIdx.x;
    const float* row = qtab + q * qstride;
    float a2 = 0.0F;
    for (uint32_t d = lane; d < kdim; d += kWave) {
        a2 = fmaf(row[d], row[d], a2);
    }
    for (int off = 32; off > 0; off >>= 1) {
        a2 += __shfl_xor(a2, off);
    }
    if (lane != 0) {
        return;
    }
    uint32_t b = bound[q];
    if (b == 0xFFFFFFFFU) {
        tau[q] = 3.0e38F;  // no bound yet: everything is a candidate (and the query will overflow)
        if (magnitude_out != nullptr) {
            magnitude_out[q] = 0.0F;
        }
        return;
    }
    float bd = ordered_to_float(b);
    float ymax = __uint_as_float(*ymax_bits);
    float cq = is_l2 ? a2 : 1.0F - (qmeta != nullptr ? qmeta[q * qmeta_stride] : 0.0F);
    float factor = is_l2 ? 2.0F : 1.0F;
    float err = factor * static_cast<float>(kdim) * 2.4e-7F * sqrtf(a2) * ymax;
    float magnitude = fabsf(bd) + fabsf(cq) + (is_l2 ? ymax * ymax : 0.0F) + factor * sqrtf(a2) * ymax;
    float t = bd - cq + err + 1.0e-6F * magnitude;
    tau[q] = t < 3.0e38F ? t : 3.0e38F;
    if (magnitude_out != nullptr) {
        magnitude_out[q] = magnitude;  // residual lists add their own terms' share to the margin (ivf_f32_kernel)
    }
}

struct RescoreArgs {
    const uint32_t* cand;
    const uint32_t* cand_cnt;
    uint32_t cap;
    uint64_t n;
    uint32_t k, S;
    uint32_t* bound;
    uint64_t* partial;
    uint32_t* partial_cnt;
    uint32_t nslots;
    uint32_t first_slot;  // the list of the first level of this call; out_slot - first_slot levels came before
    uint32_t out_slot;
    uint32_t* gate;  // per query: 1 = candidates overflowed at some level, the streaming kernel must serve the query
    // sub_lists != 0: the candidates of a query sit in sub_lists lists of sub_cap (<= gather) slots with a count each
    // (a count above sub_cap = that list overflowed); they are gathered into `gather` words of LDS.
    uint32_t sub_lists, sub_cap, gather;
    const uint4* rows;  // the codes a row per code (store.h), or null: read the tiles
    uint32_t row_granules;  // granules of a row: G, or G + 1 with the code's metadata words behind the code
};

// Words of LDS for gathered candidates: small, so that many of these one-wave workgroups share a compute unit (the
// kernel lives on memory latency), but never less than one private list.
constexpr uint32_t kRescoreGather = 1024;

// One wave per query: exact distances of its candidates by the streaming kernel's arithmetic, best k kept.
template <int KIND, int METRIC>
__global__ void __launch_bounds__(64)
rescore_kernel(ScanArgs a, RescoreArgs r) {
    extern __shared__ uint64_t keys[];
    const uint32_t lane = threadIdx.x;
    const uint32_t q = blockIdx.x;
    const uint64_t list = static_cast<uint64_t>(q) * r.nslots + r.out_slot;
    bool overflow = false;
    const uint32_t* counts = r.cand_cnt + static_cast<uint64_t>(q) * (r.sub_lists != 0 ? r.sub_lists : 1);
    if (r.sub_lists == 0) {
        overflow = as_const(counts)[0] > r.cap;
    } else {
        for (uint32_t g0 = 0; g0 < r.sub_lists; g0 += kWave) {
            const uint32_t g = g0 + lane;
            overflow = overflow || __ballot(g < r.sub_lists && as_const(counts)[g] > r.sub_cap) != 0;
        }
    }
    if (overflow || as_const(r.gate)[q] != 0) {
        // The streaming kernel will scan every tile behind the prefix for this query: the lists of the levels so
        // far must not contribute the same codes a second time.
        const uint32_t nlev = r.out_slot - r.first_slot + 1;
        if (lane < nlev) {
            r.partial_cnt[static_cast<uint64_t>(q) * r.nslots + r.first_slot + lane] = 0;
        }
        if (lane == 0) {
            r.gate[q] = 1;
        }
        return;
    }
    const uint32_t S = r.S, k = r.k;
    const uint32_t pend = selector_base(S, k);  // where the selector's pending keys start
    selector_init(keys, S, lane);
    uint32_t cnt = 0;
    uint32_t bs = __builtin_amdgcn_readfirstlane(__atomic_load_n(&r.bound[q], __ATOMIC_RELAXED));
    // Candidates arrive in no particular order, so ties are decided on whole (distance, id) keys.
    uint64_t tau = (static_cast<uint64_t>(bs) << 32) | 0xFFFFFFFFULL;
    const uint32_t qidx[1] = {q};
    const QueryRows<1> qrows = query_rows<1>(a, qidx);
    auto rescore = [&](const uint32_t* mine, uint32_t total) __attribute__((always_inline)) {
        for (uint32_t base = 0; base < total; base += kWave) {
            const bool have = base + lane < total;
            const uint32_t slot = have ? mine[base + lane] : 0U;
            const uint64_t tile = slot >> 6;
            const uint32_t ln = slot & 63;
            Acc<KIND, 1> acc;
            acc_reset(acc);
            const uint4* row = r.rows != nullptr ? r.rows + static_cast<uint64_t>(slot) * r.row_granules : nullptr;
            // A few granules are fetched before the first is used: a candidate's loads wait for memory together.
            // (sq8 l2 holds scale and query of every dimension in flight in scalar registers: two granules' worth; an sq4
            // granule is 32 dimensions.)
            constexpr uint32_t kAhead = KIND == VSAG_AMD_KIND_SQ4 ? (METRIC == VSAG_AMD_METRIC_L2 ? 1 : 2)
                                       : (KIND == VSAG_AMD_KIND_SQ8 && METRIC == VSAG_AMD_METRIC_L2 ? 2 : 4);
            for (uint32_t j0 = 0; j0 < a.G; j0 += kAhead) {
                uint4 c[kAhead];
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    const uint32_t j = j0 + u < a.G ? j0 + u : a.G - 1;
                    c[u] = row != nullptr ? row[j] : a.tiles[(tile * a.G + j) * kWave + ln];
                }
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    if (j0 + u < a.G) {
                        accumulate_granule<KIND, METRIC, 1>(a, qrows, j0 + u, c[u], acc);
                    }
                }
            }
            float d[1];
            if (r.row_granules > a.G) {
                // The metadata words of the code sit behind it in the row: the same words in the same arithmetic, but one
                // run of memory per candidate instead of a line per word.
                ScanArgs b = a;
                b.meta = reinterpret_cast<const uint32_t*>(row + a.G);
                b.meta_stride = 1;
                finish_distances<KIND, METRIC, 1>(b, qidx, 0, acc, d);
            } else {
                finish_distances<KIND, METRIC, 1>(a, qidx, slot, acc, d);
            }
            const uint64_t key = make_key(d[0], slot);
            bool pass = have && slot < r.n && key <= tau;
            uint64_t mask = __ballot(pass);
            if (mask != 0) {
                uint32_t np = __popcll(mask);
                if (pend + cnt + np > S) {
                    uint64_t th = selector_flush(keys, S, k, cnt, lane);
                    cnt = 0;
                    uint32_t b = lower_shared(&r.bound[q], static_cast<uint32_t>(th >> 32), lane);
                    uint64_t shared_tau = (static_cast<uint64_t>(b) << 32) | 0xFFFFFFFFULL;
                    tau = th < shared_tau ? th : shared_tau;
                }
                if (pass) {
                    keys[pend + cnt + mask_rank(mask)] = key;
                }
                cnt += np;
            }
        }
    };
    if (r.sub_lists == 0) {
        rescore(r.cand + static_cast<uint64_t>(q) * r.cap, as_const(counts)[0]);
    } else {
        // Gather the private lists of the query behind the selector -- a lane per list, offsets by a wave scan -- and
        // rescore whenever the next lists might not fit (usually once, at the end: full waves of candidates).  64 lists
        // go in one round when what they hold fits; a round of fuller lists goes in pieces that fit even when full.
        uint32_t* flat = reinterpret_cast<uint32_t*>(keys + r.S);
        const uint32_t* lists = r.cand + static_cast<uint64_t>(q) * r.sub_lists * r.sub_cap;
        uint32_t piece = r.gather / r.sub_cap;
        piece = piece > kWave ? kWave : (piece == 0 ? 1 : piece);
        uint32_t fill = 0;
        auto gather = [&](uint32_t g, uint32_t c) {
            // c = this lane's share (0: none); returns after the lanes' entries are in flat[fill ...].
            uint32_t incl = c;
            for (int off = 1; off < 64; off <<= 1) {
                uint32_t o = __shfl_up(incl, off);
                incl += lane >= static_cast<uint32_t>(off) ? o : 0U;
            }
            const uint32_t sum = __shfl(incl, 63);
            if (sum == 0) {
                return;
            }
            if (fill + sum > r.gather) {
                wave_lds_fence();
                rescore(flat, fill);
                fill = 0;
                wave_lds_fence();  // what was gathered has been read
            }
            const uint32_t at = fill + incl - c;
            const uint32_t* mine = lists + static_cast<uint64_t>(g) * r.sub_cap;
            // Four loads in flight per lane.
            for (uint32_t i = 0; i < c; i += 4) {
                uint32_t v[4];
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) {
                    v[j] = i + j < c ? as_const(mine)[i + j] : 0U;
                }
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) {
                    if (i + j < c) {
                        flat[at + i + j] = v[j];
                    }
                }
            }
            fill += sum;
        };
        // The counts of four rounds are asked for together: a query with thousands of (mostly empty) private lists
        // would otherwise wait for memory once per 64 of them.
        auto round = [&](uint32_t g, uint32_t c) {
            uint32_t total = c;
            for (int off = 32; off > 0; off >>= 1) {
                total += __shfl_xor(total, off);
            }
            if (total == 0) {
                return;
            }
            if (total <= r.gather) {
                gather(g, c);
            } else {
                for (uint32_t b0 = 0; b0 < kWave; b0 += piece) {
                    gather(g, lane >= b0 && lane < b0 + piece ? c : 0U);
                }
            }
        };
        for (uint32_t g4 = 0; g4 < r.sub_lists; g4 += 4 * kWave) {
            const uint32_t ga = g4 + lane, gb = ga + kWave, gc = gb + kWave, gd = gc + kWave;
            const uint32_t ca = ga < r.sub_lists ? as_const(counts)[ga] : 0U;
            const uint32_t cb = gb < r.sub_lists ? as_const(counts)[gb] : 0U;
            const uint32_t cc = gc < r.sub_lists ? as_const(counts)[gc] : 0U;
            const uint32_t cd = gd < r.sub_lists ? as_const(counts)[gd] : 0U;
            // (one call in a loop that stays a loop: four calls would make the rounds a function with a stack frame)
#pragma nounroll
            for (uint32_t u = 0; u < 4; ++u) {
                round(ga + u * kWave, u == 0 ? ca : (u == 1 ? cb : (u == 2 ? cc : cd)));
            }
        }
        wave_lds_fence();
        rescore(flat, fill);
    }
    wave_lds_fence();
    bs = __builtin_amdgcn_readfirstlane(__atomic_load_n(&r.bound[q], __ATOMIC_RELAXED));
    uint32_t kept = pend + cnt;
    uint32_t admitted = selector_count_admitted(keys, kept, bs, lane);
    if (admitted > k) {
        uint64_t th = selector_flush(keys, S, k, cnt, lane);
        bs = lower_shared(&r.bound[q], static_cast<uint32_t>(th >> 32), lane);
        kept = k;
        admitted = selector_count_admitted(keys, kept, bs, lane);
    }
    if (lane == 0) {
        r.partial_cnt[list] = admitted;
    }
    if (admitted != 0) {
        selector_copy_admitted(keys, kept, bs, r.partial + list * k, lane);
    }
}

// Posting lists: the matrix-core pass over sq8 lists (prefilter_i8.hip, ivf_sq8_i8_kernel) leaves, per (query, list)
// pair, per_pair private lists of tile slots in the partial lists of an ivf scan.  One wave per query turns the
// records of probe columns [p0, nprobe) into (distance, id) keys by the streaming kernel's arithmetic, in place: the
// records of 64 lists (or, when those hold many, of as many lists as always fit) are gathered in LDS, a lane computes
// a record's key, and the lane that owns a list writes the keys that count back to its front.  Records of empty slots
// and of distances beyond the query's bound are dropped.
struct IvfRescoreArgs {
    uint64_t* partial;
    uint32_t* partial_cnt;
    uint32_t k;  // capacity of a private list, at most kIvfRescoreGather
    uint32_t nprobe, p0, per_pair;
    const uint32_t* ids;
    const uint32_t* bound;
    // Residual lists (ivf.hip, IvfArgs): the slot's bias and the pair's term come off the distance, in the streaming
    // kernel's order.  res_term null: no residual.
    const float* res_bias;
    const float* res_term;
};

constexpr uint32_t kIvfRescoreGather = 1024;

template <int KIND, int METRIC>
__global__ void __launch_bounds__(64)
ivf_rescore_kernel(ScanArgs a, IvfRescoreArgs r) {
    __shared__ uint32_t where[kIvfRescoreGather];
    __shared__ uint64_t fkey[kIvfRescoreGather];
    const uint32_t lane = threadIdx.x;
    const uint32_t q = blockIdx.x;
    const uint32_t lists = (r.nprobe - r.p0) * r.per_pair;
    const uint64_t base = (static_cast<uint64_t>(q) * r.nprobe + r.p0) * r.per_pair;
    uint64_t* mine = r.partial + base * r.k;
    uint32_t* counts = r.partial_cnt + base;
    const uint32_t bound = as_const(r.bound)[q];
    const uint32_t qidx[1] = {q};
    const QueryRows<1> qrows = query_rows<1>(a, qidx);
    uint32_t piece = kIvfRescoreGather / r.k;
    piece = piece > kWave ? kWave : piece;
    constexpr uint64_t kDropped = ~0ULL;
    auto round = [&](uint32_t g, uint32_t c) {
        // c = records of this lane's list g that take part (0: none).
        uint32_t incl = c;
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(incl, off);
            incl += lane >= static_cast<uint32_t>(off) ? o : 0U;
        }
        const uint32_t sum = __shfl(incl, 63);
        if (sum == 0) {
            return;
        }
        const uint32_t at = incl - c;
        for (uint32_t i = 0; i < c; ++i) {
            where[at + i] = g * r.k + i;
        }
        wave_lds_fence();
        for (uint32_t e0 = 0; e0 < sum; e0 += kWave) {
            const bool have = e0 + lane < sum;
            const uint32_t slot = have ? static_cast<uint32_t>(mine[where[e0 + lane]]) : 0U;
            const uint64_t tile = slot >> 6;
            const uint32_t ln = slot & 63;
            Acc<KIND, 1> acc;
            acc_reset(acc);
            constexpr uint32_t kAhead = KIND == VSAG_AMD_KIND_SQ4 ? (METRIC == VSAG_AMD_METRIC_L2 ? 1 : 2)
                                       : (KIND == VSAG_AMD_KIND_SQ8 && METRIC == VSAG_AMD_METRIC_L2 ? 2 : 4);
            for (uint32_t j0 = 0; j0 < a.G; j0 += kAhead) {
                uint4 c4[kAhead];
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    const uint32_t j = j0 + u < a.G ? j0 + u : a.G - 1;
                    c4[u] = a.tiles[(tile * a.G + j) * kWave + ln];
                }
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    if (j0 + u < a.G) {
                        accumulate_granule<KIND, METRIC, 1>(a, qrows, j0 + u, c4[u], acc);
                    }
                }
            }
            float d[1];
            finish_distances<KIND, METRIC, 1>(a, qidx, slot, acc, d);
            if (r.res_term != nullptr && have) {
                // list g of the query belongs to its pair p0 + g / per_pair
                const uint32_t gl = where[e0 + lane] / r.k;
                const float bias = r.res_bias != nullptr ? r.res_bias[slot] : 0.0F;
                d[0] = (d[0] - bias) - r.res_term[static_cast<uint64_t>(q) * r.nprobe + r.p0 + gl / r.per_pair];
            }
            if (have) {
                const uint32_t id = as_const(r.ids)[slot];
                fkey[e0 + lane] =
                    id != VSAG_AMD_INVALID_ID && float_to_ordered(d[0]) <= bound ? make_key(d[0], id) : kDropped;
            }
        }
        wave_lds_fence();
        if (c != 0) {
            uint32_t kept = 0;
            for (uint32_t i = 0; i < c; ++i) {
                const uint64_t key = fkey[at + i];
                if (key != kDropped) {
                    mine[static_cast<uint64_t>(g) * r.k + kept++] = key;
                }
            }
            counts[g] = kept;
        }
        wave_lds_fence();  // the next round writes the same LDS
    };
    for (uint32_t g0 = 0; g0 < lists; g0 += kWave) {
        const uint32_t g = g0 + lane;
        const uint32_t c = g < lists ? as_const(counts)[g] : 0U;
        uint32_t total = c;
        for (int off = 32; off > 0; off >>= 1) {
            total += __shfl_xor(total, off);
        }
        if (total == 0) {
            continue;
        }
        if (total <= kIvfRescoreGather) {
            round(g, c);
        } else {
            for (uint32_t b0 = 0; b0 < kWave; b0 += piece) {
                round(g, lane >= b0 && lane < b0 + piece ? c : 0U);
            }
        }
    }
}

uint32_t
ivf_rescore_capacity() {
    return kIvfRescoreGather;
}

int
launch_ivf_rescore(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
                   uint32_t per_pair, uint64_t* partial, uint32_t* partial_cnt, const uint32_t* bound, const float* res_term,
                   hipStream_t st) {
    if ((s->kind != VSAG_AMD_KIND_SQ8 && s->kind != VSAG_AMD_KIND_SQ4 && s->kind != VSAG_AMD_KIND_RABITQ &&
         s->kind != VSAG_AMD_KIND_FP32) ||
        kcand > kIvfRescoreGather || s->ids_dev == nullptr) {
        return fail(VSAG_AMD_INVALID_ARGUMENT,
                    "rescoring of list records: fp32, sq8, sq4 or rabitq lists with kcand <= %u only", kIvfRescoreGather);
    }
    IvfRescoreArgs r{};
    r.partial = partial;
    r.partial_cnt = partial_cnt;
    r.k = kcand;
    r.nprobe = nprobe;
    r.p0 = p0;
    r.per_pair = per_pair;
    r.ids = s->ids_dev;
    r.bound = bound;
    r.res_term = res_term;
    r.res_bias = res_term != nullptr ? s->residual_bias_dev : nullptr;
    const dim3 grid(static_cast<uint32_t>(nq));
    if (s->kind == VSAG_AMD_KIND_FP32) {
        // (cosine stores hold normalised vectors and scan as inner product)
        if (s->metric == VSAG_AMD_METRIC_L2) {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_FP32, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), 0, st, a, r);
        } else {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_FP32, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), 0, st, a, r);
        }
    } else if (s->kind == VSAG_AMD_KIND_RABITQ) {
        if (s->metric == VSAG_AMD_METRIC_L2) {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_RABITQ, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), 0, st, a, r);
        } else {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_RABITQ, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), 0, st, a, r);
        }
    } else if (s->kind == VSAG_AMD_KIND_SQ4) {
        if (s->metric == VSAG_AMD_METRIC_L2) {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_SQ4, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), 0, st, a, r);
        } else {
            hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_SQ4, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), 0, st, a, r);
        }
    } else if (s->metric == VSAG_AMD_METRIC_L2) {
        hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_SQ8, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), 0, st, a, r);
    } else {
        hipLaunchKernelGGL((ivf_rescore_kernel<VSAG_AMD_KIND_SQ8, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), 0, st, a, r);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

// ---- fp32 (and sq8 of any dimension) posting lists against large batches ------------------------------------------
// The contraction of prefilter_kernel over the (query, list) pairs of an ivf search that the streaming kernel has already
// given a bound (the probe columns behind the nearest list; ivf_i8.hip describes the work split this kernel shares: the
// pairs are grouped by list, a work item = a chunk of a list's tiles x up to 128 of the pairs that probe the list).
// The B operand rows of an item are whatever queries probe the list, fetched through the pair table.  What passes is
// recorded as a tile slot in the private list (pair, chunk, which 64 codes of the 128-code tile) -- the lists the
// streaming kernel's partial results use -- and turned into a (distance, id) key by ivf_rescore_kernel.
constexpr uint32_t kIvfF32Pairs = PN;
constexpr uint32_t kIvfF32ChunkTiles = 32;  // as ivf_i8.hip: kIvfI8ChunkTiles, kIvfI8Chunks
constexpr uint32_t kIvfF32Chunks = 4;

struct IvfF32Args {
    const uint4* tiles;
    uint32_t G;
    const float* scale;             // sq8, l2: y_d = c_d * scale_d; null: y_d = c_d
    const float* qtab;
    uint32_t qstride;
    uint32_t kdim;
    const float* term;              // per slot |y|^2
    float term_factor, dot_factor;  // as PrefilterArgs
    const float* tau;               // per query
    // Residual lists: distance = (base - bias of the slot) - term of the pair, so the bias joins the code's term, the
    // pair's term the threshold, and the margin grows by their rounding: res_margin x (the query's magnitudes +
    // |term| + res_bias_max).  res_term null: no residual.
    const float* res_bias;          // per slot, or null (inner product)
    const float* res_term;          // per pair (query * nprobe + column)
    const float* magnitude;         // per query, from prefilter_tau_kernel
    const uint32_t* ymax_bits;      // the largest norm among the stored vectors
    float res_cmax;                 // the largest norm among the lists' centroids
    const uint32_t* ids;            // per slot; the padding behind a list's last code holds no id and never passes
    const uint32_t* list_tile;      // per list: first tile, end tile
    const uint32_t* pair_off;       // pairs of list b: sorted_pair[pair_off[b] .. pair_off[b + 1])
    const uint32_t* item_off;       // items of list b: item_off[b] .. item_off[b + 1]
    const uint32_t* sorted_pair;    // query * nprobe + column
    uint32_t nlist, nprobe;
    uint64_t nq;
    uint32_t k;                     // records per private list
    uint64_t* partial;
    uint32_t* partial_cnt;          // zero before the launch; may end above k (overflow: the query is gated)
    uint32_t* gate;                 // nq + 2 words as in ivf_i8.hip
};

template <int KIND>
__global__ void __launch_bounds__(256, 3)
ivf_f32_kernel(IvfF32Args p) {
    __shared__ PfStage stage[1];
    __shared__ float code_term[PM];
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
    uint32_t chunks = (list_end - list_begin + kIvfF32ChunkTiles - 1) / kIvfF32ChunkTiles;
    chunks = chunks < kIvfF32Chunks ? chunks : kIvfF32Chunks;
    if (chunks == 0) {
        return;
    }
    const uint32_t per = (list_end - list_begin + chunks - 1) / chunks;
    const uint32_t chunk = (item - ioff[b]) % chunks;
    const uint32_t group = (item - ioff[b]) / chunks;
    uint32_t tile_begin = list_begin + chunk * per;
    tile_begin = tile_begin < list_end ? tile_begin : list_end;
    const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
    const uint32_t pbeg = as_const(p.pair_off)[b] + group * kIvfF32Pairs;
    const uint32_t pend = as_const(p.pair_off)[b + 1];
    const uint32_t mtiles = (tile_end - tile_begin + 1) / 2;
    if (mtiles == 0 || pbeg >= pend) {
        return;
    }
    const uint32_t ktiles = (p.kdim + PK - 1) / PK;

    // Query loader roles as in prefilter_kernel; the rows are the queries of this item's pairs.
    uint32_t qc[2];
    uint64_t qsrc[2];
    uint32_t qrow[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint32_t idx = tid + 256 * r;
        qrow[r] = idx >> 2;
        qc[r] = idx & 3;
        const uint32_t at = pbeg + qrow[r];
        qsrc[r] = at < pend ? as_const(p.sorted_pair)[at] / p.nprobe : p.nq;  // p.nq: no such row, zeros
    }
    float tau_n[2];
    uint32_t pair_n[2], query_n[2];
    bool live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t at = pbeg + wn * 64 + j * 32 + l32;
        live[j] = at < pend;
        pair_n[j] = live[j] ? as_const(p.sorted_pair)[at] : 0U;
        query_n[j] = pair_n[j] / p.nprobe;
        tau_n[j] = live[j] ? p.tau[query_n[j]] : -__builtin_inff();
        if (p.res_term != nullptr && live[j]) {
            const float rt = p.res_term[pair_n[j]];
            // |bias| = |2 <c, y> + |c|^2| (l2; inner product has none)
            const float res_bias_max =
                p.res_bias != nullptr ? (2.0F * __uint_as_float(*p.ymax_bits) + p.res_cmax) * p.res_cmax : 0.0F;
            // five more roundings between this test and the streaming result (the slot's term less its bias, the
            // threshold plus the pair's term, and the two subtractions of the streaming kernel): 2e-6 of the magnitudes
            // is several times their sum
            tau_n[j] = tau_n[j] + rt + 2.0e-6F * (p.magnitude[query_n[j]] + fabsf(rt) + res_bias_max);
        }
    }

    const uint32_t crow = tid & 127;
    const uint32_t cpart = tid >> 7;
    auto code_granule = [&](uint32_t mt, uint32_t j) {
        const uint32_t tile = tile_begin + 2 * mt + (crow >> 6);
        if (tile < tile_end && j < p.G) {
            return p.tiles[(static_cast<uint64_t>(tile) * p.G + j) * kWave + (crow & 63)];
        }
        return make_uint4(0, 0, 0, 0);
    };
    constexpr int kCodeRegs = KIND == VSAG_AMD_KIND_SQ8 ? 1 : 4;
    auto fetch_codes = [&](uint32_t mt, uint32_t kt, uint4 (&regs)[kCodeRegs]) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
            regs[0] = code_granule(mt, 2 * kt + cpart);
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                regs[2 * r] = code_granule(mt, 8 * kt + 2 * (cpart + 2 * r));
                regs[2 * r + 1] = code_granule(mt, 8 * kt + 2 * (cpart + 2 * r) + 1);
            }
        }
    };
    auto as_floats = [](uint4 v) {
        return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    };
    auto park_codes = [&](float4* plane, uint32_t kt, const uint4 (&regs)[kCodeRegs]) {
        if constexpr (KIND == VSAG_AMD_KIND_SQ8) {
            const uint32_t w[4] = {regs[0].x, regs[0].y, regs[0].z, regs[0].w};
            const uint32_t d0 = PK * kt + 16 * cpart;
            float4 v[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                v[m] = make_float4(static_cast<float>(w[m] & 0xffU), static_cast<float>((w[m] >> 8) & 0xffU),
                                   static_cast<float>((w[m] >> 16) & 0xffU), static_cast<float>(w[m] >> 24));
                if (p.scale != nullptr && d0 + 16 <= p.kdim) {
                    float4 sc = *reinterpret_cast<const float4*>(p.scale + d0 + 4 * m);
                    v[m].x *= sc.x;
                    v[m].y *= sc.y;
                    v[m].z *= sc.z;
                    v[m].w *= sc.w;
                }
            }
            pf_stage_store8(plane, crow, 2 * cpart, v[0], v[1]);
            pf_stage_store8(plane, crow, 2 * cpart + 1, v[2], v[3]);
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                pf_stage_store8(plane, crow, cpart + 2 * r, as_floats(regs[2 * r]), as_floats(regs[2 * r + 1]));
            }
        }
    };
    uint4 rc[kCodeRegs];
    float4 rq[4];
    auto fetch_queries = [&](uint32_t kt) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            rq[2 * r] = pf_query_chunk(p.qtab, qsrc[r], p.nq, PK * kt + 8 * qc[r], p.qstride);
            rq[2 * r + 1] = pf_query_chunk(p.qtab, qsrc[r], p.nq, PK * kt + 8 * qc[r] + 4, p.qstride);
        }
    };
    auto park_queries = [&](float4* plane) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            pf_stage_store8(plane, qrow[r], qc[r], rq[2 * r], rq[2 * r + 1]);
        }
    };
    fetch_codes(0, 0, rc);
    fetch_queries(0);
    for (uint32_t mt = 0; mt < mtiles; ++mt) {
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
        const uint64_t slot0 = (static_cast<uint64_t>(tile_begin) + 2 * mt) * kWave;
        park_codes(stage[0].a, 0, rc);
        park_queries(stage[0].b);
        float my_term = 0.0F;
        if (tid < PM) {
            // (a padding slot is all zeros: under inner product, and with a residual bias, that is a good distance)
            const bool real = tile_begin + 2 * mt + (tid >> 6) < tile_end && p.ids[slot0 + tid] != VSAG_AMD_INVALID_ID;
            my_term = real ? p.term_factor * p.term[slot0 + tid] : __builtin_inff();
            if (real && p.res_bias != nullptr) {
                my_term -= p.res_bias[slot0 + tid];
            }
        }
        __syncthreads();
        for (uint32_t kt = 0; kt < ktiles; ++kt) {
            if (kt + 1 < ktiles) {
                fetch_codes(mt, kt + 1, rc);
                fetch_queries(kt + 1);
            } else if (mt + 1 < mtiles) {
                fetch_codes(mt + 1, 0, rc);
                fetch_queries(0);
            }
            const float4* pa = stage[0].a + half * 4 * kPfPlane + wm * 64 + l32;
            const float4* pb = stage[0].b + half * 4 * kPfPlane + wn * 64 + l32;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float4 a0 = pa[c * kPfPlane];
                float4 a1 = pa[c * kPfPlane + 32];
                float4 b0 = pb[c * kPfPlane];
                float4 b1 = pb[c * kPfPlane + 32];
                const float av0[4] = {a0.x, a0.y, a0.z, a0.w};
                const float av1[4] = {a1.x, a1.y, a1.z, a1.w};
                const float bv0[4] = {b0.x, b0.y, b0.z, b0.w};
                const float bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv0[e], acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv1[e], acc[0][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv0[e], acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv1[e], acc[1][1], 0, 0, 0);
                }
            }
            if (kt + 1 == ktiles && tid < PM) {
                code_term[tid] = my_term;
            }
            __syncthreads();
            if (kt + 1 < ktiles) {
                park_codes(stage[0].a, kt + 1, rc);
                park_queries(stage[0].b);
                __syncthreads();
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t hits = 0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    const float v = code_term[ml] + p.dot_factor * acc[i][j][e];
                    hits |= (v <= tau_n[j] ? 1U : 0U) << (16 * i + e);
                }
            }
            if (hits != 0 && live[j]) {
                const uint64_t list = (static_cast<uint64_t>(pair_n[j]) * kIvfF32Chunks + chunk) * 2 + wm;
                while (hits != 0) {
                    const uint32_t bit = static_cast<uint32_t>(__builtin_ctz(hits));
                    hits &= hits - 1;
                    const uint32_t i = bit >> 4, e = bit & 15;
                    const uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
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

bool
ivf_f32_supports(const vsag_amd_store* s) {
    return (s->kind == VSAG_AMD_KIND_FP32 || s->kind == VSAG_AMD_KIND_SQ8) && s->nlist > 0 && s->pf_term != nullptr &&
           s->pf_ymax != nullptr && s->ids_dev != nullptr &&
           (s->residual_centroids_dev == nullptr || s->metric != VSAG_AMD_METRIC_COSINE);
}

uint32_t
ivf_f32_pairs_per_item() {
    return kIvfF32Pairs;
}

// Thresholds from the bounds (tau: nq floats), then the candidates of probe columns [p0, nprobe) grouped by list
// (pair_off, sorted_pair; item_off counted with ivf_f32_pairs_per_item() pairs per item) into the private lists
// (pair * 8 + chunk * 2 + half tile) of kcand records in `partial`; partial_cnt zero before.  gate: nq + 2 words.
int
launch_ivf_f32(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
               const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, float* tau,
               uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const float* res_term, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const bool sq8 = s->kind == VSAG_AMD_KIND_SQ8;
    // tau: nq thresholds, then (residual lists) nq magnitudes behind a spare word
    hipLaunchKernelGGL(prefilter_tau_kernel, dim3(static_cast<uint32_t>(nq)), dim3(kWave), 0, st,
                       reinterpret_cast<const float*>(a.qtab), a.qstride, s->dpad, sq8 && !l2 ? a.qmeta : nullptr,
                       a.qmeta_stride, l2 ? 1 : 0, bound, s->pf_ymax, nq, tau, res_term != nullptr ? tau + nq + 1 : nullptr);
    IvfF32Args p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.scale = sq8 && l2 ? s->scale_dev : nullptr;
    p.qtab = reinterpret_cast<const float*>(a.qtab);
    p.qstride = a.qstride;
    p.kdim = s->dpad;
    p.term = s->pf_term;
    p.term_factor = l2 ? 1.0F : 0.0F;
    p.dot_factor = l2 ? -2.0F : -1.0F;
    p.tau = tau;
    if (res_term != nullptr) {
        p.res_term = res_term;
        p.res_bias = s->residual_bias_dev;
        p.magnitude = tau + nq + 1;
        p.ymax_bits = s->pf_ymax;
        p.res_cmax = s->residual_cmax;
    }
    p.ids = s->ids_dev;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.nq = nq;
    p.k = kcand;
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kIvfF32Pairs)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfF32Chunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    if (sq8) {
        hipLaunchKernelGGL(ivf_f32_kernel<VSAG_AMD_KIND_SQ8>, grid, dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL(ivf_f32_kernel<VSAG_AMD_KIND_FP32>, grid, dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    // (Counts run past the capacity where a list overflowed; those lists are emptied with their pair's, or their
    // query's, before anything reads them: launch_ivf_clear_gated.)
    return 0;
}

// ------------------------------------------------------------------ host side
bool prefilter_rb_supports(const vsag_amd_store* s);
int launch_prefilter_rb(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                        const uint32_t* bound, uint8_t* scratch, uint32_t* cand, uint32_t* cand_cnt, uint32_t sub_lists,
                        uint32_t sub_cap, hipStream_t st);

bool prefilter_i8_supports(const vsag_amd_store* s);
bool prefilter_h16_supports(const vsag_amd_store* s);
int launch_prefilter_h16(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                         const uint32_t* bound, float* tau, uint8_t* scratch, uint32_t* cand, uint32_t* cand_cnt,
                         uint32_t cap, hipStream_t st);

bool
prefilter_supports(const vsag_amd_store* s) {
    if (prefilter_rb_supports(s)) {
        return true;
    }
    if (s->kind == VSAG_AMD_KIND_SQ4) {
        return prefilter_i8_supports(s) || prefilter_h16_supports(s);  // int8 up to 128 dimensions, fp16 beyond
    }
    if (s->kind == VSAG_AMD_KIND_SQ8_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4_UNIFORM) {
        return prefilter_i8_supports(s);  // the int8 matrix cores or nothing
    }
    return s->nlist == 0 && (s->kind == VSAG_AMD_KIND_FP32 || s->kind == VSAG_AMD_KIND_SQ8) && s->pf_term != nullptr;
}

// sq8_uniform: the per-code term of the int8 test, from the code's stored scalar (prefilter_i8.hip).
__global__ void __launch_bounds__(256)
uniform_term_kernel(const uint32_t* meta, uint64_t first, uint64_t count, int is_l2, float lb, float* term) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) {
        const float m = __uint_as_float(meta[first + i]);
        term[first + i] = is_l2 ? m : -(lb * m);
    }
}

// |y|^2 for freshly appended codes (y as the contraction sees it: scaled codes for sq8 l2, raw code values
// for sq8 ip, the stored vector for fp32).
int
launch_code_terms(vsag_amd_store* s, uint64_t first, uint64_t count, hipStream_t st) {
    if (count == 0 || s->pf_term == nullptr) {
        return 0;
    }
    dim3 grid(static_cast<uint32_t>(div_up(count, 256)));
    if (s->kind == VSAG_AMD_KIND_SQ8_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4_UNIFORM) {
        hipLaunchKernelGGL(uniform_term_kernel, grid, dim3(256), 0, st, s->meta, first, count,
                           s->metric == VSAG_AMD_METRIC_L2 ? 1 : 0, s->ulb, s->pf_term);
    } else if (s->kind == VSAG_AMD_KIND_SQ8) {
        const float* scale = s->metric == VSAG_AMD_METRIC_L2 ? s->scale_dev : nullptr;
        hipLaunchKernelGGL(code_term_kernel<VSAG_AMD_KIND_SQ8>, grid, dim3(256), 0, st, s->tiles, s->G, scale, first,
                           count, s->pf_term, s->pf_ymax);
    } else if (s->kind == VSAG_AMD_KIND_SQ4) {
        const float* scale = s->metric == VSAG_AMD_METRIC_L2 ? s->scale_dev : nullptr;
        hipLaunchKernelGGL(code_term_kernel<VSAG_AMD_KIND_SQ4>, grid, dim3(256), 0, st, s->tiles, s->G, scale, first,
                           count, s->pf_term, s->pf_ymax);
    } else {
        hipLaunchKernelGGL(code_term_kernel<VSAG_AMD_KIND_FP32>, grid, dim3(256), 0, st, s->tiles, s->G,
                           static_cast<const float*>(nullptr), first, count, s->pf_term, s->pf_ymax);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

template <int KIND>
static void
launch_rescore_m(int metric, dim3 grid, size_t lds, hipStream_t st, const ScanArgs& a, const RescoreArgs& r) {
    if (metric == VSAG_AMD_METRIC_L2) {
        hipLaunchKernelGGL((rescore_kernel<KIND, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), lds, st, a, r);
    } else {
        hipLaunchKernelGGL((rescore_kernel<KIND, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), lds, st, a, r);
    }
}

int launch_prefilter_i8(const vsag_amd_store* s, const float* qtab, uint32_t qstride, const float* qmeta,
                        uint32_t qmeta_stride, uint64_t nq, uint64_t tile_begin, uint64_t tile_end,
                        const uint32_t* bound, uint8_t* q8, float* u, uint32_t* tau, uint32_t* cand, uint32_t* cand_cnt,
                        uint32_t sub_lists, uint32_t sub_cap, bool first_level, const float* merged_dists, uint32_t k,
                        uint32_t* bound_rw, hipStream_t st);

// Step 3 of the header comment: exact distances of the collected candidates.
static int
launch_rescore(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t k, uint32_t S, uint32_t* bound,
               const uint32_t* cand, const uint32_t* cand_cnt, uint32_t cap, uint32_t sub_lists, uint32_t sub_cap,
               uint64_t* partial, uint32_t* partial_cnt, uint32_t nslots, uint32_t first_slot, uint32_t out_slot,
               uint32_t* gate, hipStream_t st) {
    RescoreArgs r{};
    r.first_slot = first_slot;
    r.cand = cand;
    r.cand_cnt = cand_cnt;
    r.cap = cap;
    r.n = s->n;
    r.k = k;
    r.S = S;
    r.bound = bound;
    r.partial = partial;
    r.partial_cnt = partial_cnt;
    r.nslots = nslots;
    r.out_slot = out_slot;
    r.gate = gate;
    r.sub_lists = sub_lists;
    r.sub_cap = sub_cap;
    r.gather = std::max(kRescoreGather, sub_cap);
    r.rows = s->rows;
    r.row_granules = s->row_granules;
    dim3 rgrid(static_cast<uint32_t>(nq));
    const size_t lds = S * 8 + (sub_lists != 0 ? r.gather * 4 : 0);
    if (s->kind == VSAG_AMD_KIND_SQ8) {
        launch_rescore_m<VSAG_AMD_KIND_SQ8>(s->metric, rgrid, lds, st, a, r);
    } else if (s->kind == VSAG_AMD_KIND_SQ4) {
        launch_rescore_m<VSAG_AMD_KIND_SQ4>(s->metric, rgrid, lds, st, a, r);
    } else if (s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
        launch_rescore_m<VSAG_AMD_KIND_SQ8_UNIFORM>(s->metric, rgrid, lds, st, a, r);
    } else if (s->kind == VSAG_AMD_KIND_SQ4_UNIFORM) {
        launch_rescore_m<VSAG_AMD_KIND_SQ4_UNIFORM>(s->metric, rgrid, lds, st, a, r);
    } else if (s->kind == VSAG_AMD_KIND_RABITQ) {
        launch_rescore_m<VSAG_AMD_KIND_RABITQ>(s->metric, rgrid, lds, st, a, r);
    } else {
        launch_rescore_m<VSAG_AMD_KIND_FP32>(s->metric, rgrid, lds, st, a, r);
    }
    VA_HIP(hipGetLastError());
    return 0;
}


// Steps 2 and 3 of the header comment for tiles [tile_begin, tile_end); the exact prefix scan has already
// left its bounds in `bound`.  Writes one partial list per query (out_slot) and raises the overflow flags.
int
launch_prefilter(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t k, uint32_t S, uint64_t tile_begin,
                 uint64_t tile_end, uint32_t* bound, float* tau, uint32_t* cand, uint32_t* cand_cnt, uint32_t cap,
                 uint64_t* partial, uint32_t* partial_cnt, uint32_t nslots, uint32_t first_slot, uint32_t out_slot,
                 uint32_t* gate, uint8_t* q8, float* q8_u, uint32_t sub_lists, uint32_t sub_cap,
                 const float* merged_dists, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    const bool sq8 = s->kind == VSAG_AMD_KIND_SQ8;
    if (s->kind == VSAG_AMD_KIND_RABITQ) {
        // 1-bit codes against 4-bit queries on the int8 matrix cores (prefilter_rb.hip); q8 is its scratch.
        VA_TRY(launch_prefilter_rb(s, a, nq, tile_begin, tile_end, bound, q8, cand, cand_cnt, sub_lists, sub_cap, st));
        return launch_rescore(s, a, nq, k, S, bound, cand, cand_cnt, 0, sub_lists, sub_cap, partial, partial_cnt, nslots,
                              first_slot, out_slot, gate, st);
    }
    if (q8 != nullptr && prefilter_h16_supports(s)) {
        // sq8 beyond 128 dimensions: the fp16 matrix cores pre-select (prefilter_h16.hip); q8 is its scratch.
        VA_TRY(launch_prefilter_h16(s, a, nq, tile_begin, tile_end, bound, tau, q8, cand, cand_cnt, cap, st));
        return launch_rescore(s, a, nq, k, S, bound, cand, cand_cnt, cap, 0, 0, partial, partial_cnt, nslots, first_slot,
                              out_slot, gate, st);
    }
    if (q8 != nullptr) {
        // At most 128 dimensions of sq8: the int8 matrix cores pre-select (prefilter_i8.hip).
        VA_TRY(launch_prefilter_i8(s, reinterpret_cast<const float*>(a.qtab), a.qstride, a.qmeta, a.qmeta_stride, nq,
                                   tile_begin, tile_end, bound, q8, q8_u, reinterpret_cast<uint32_t*>(tau), cand,
                                   cand_cnt, sub_lists, sub_cap, out_slot == first_slot, merged_dists, k, bound, st));
        return launch_rescore(s, a, nq, k, S, bound, cand, cand_cnt, 0, sub_lists, sub_cap, partial, partial_cnt, nslots,
                              first_slot, out_slot, gate, st);
    }
    hipLaunchKernelGGL(prefilter_tau_kernel, dim3(static_cast<uint32_t>(nq)), dim3(kWave), 0, st,
                       reinterpret_cast<const float*>(a.qtab), a.qstride, s->dpad, sq8 && !l2 ? a.qmeta : nullptr,
                       a.qmeta_stride, l2 ? 1 : 0, bound, s->pf_ymax, nq, tau);
    PrefilterArgs p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.tile_begin = tile_begin;
    p.tile_end = tile_end;
    p.n = s->n;
    p.scale = sq8 && l2 ? s->scale_dev : nullptr;
    p.qtab = reinterpret_cast<const float*>(a.qtab);
    p.qstride = a.qstride;
    p.nq = nq;
    p.kdim = s->dpad;
    p.term = s->pf_term;
    p.term_factor = l2 ? 1.0F : 0.0F;
    p.dot_factor = l2 ? -2.0F : -1.0F;
    p.tau = tau;
    p.cand = cand;
    p.cand_cnt = cand_cnt;
    p.cap = cap;
    const uint64_t mtiles = (tile_end - tile_begin + 1) / 2;
    const uint64_t qtiles = div_up(nq, static_cast<uint64_t>(PN));
    // At most six workgroups per compute unit (two rounds of the three that fit) and not one more: a few left over
    // would run a third round alone.  A group walks every groups-th code tile.
    uint64_t groups = static_cast<uint64_t>(device_cu_count()) * 6 / qtiles;
    groups = std::max<uint64_t>(1, std::min<uint64_t>(groups, mtiles));
    p.groups = static_cast<uint32_t>(groups);
    dim3 grid(p.groups, static_cast<uint32_t>(qtiles));
    timing_begin(st);
    if (sq8) {
        hipLaunchKernelGGL(prefilter_kernel<VSAG_AMD_KIND_SQ8>, grid, dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL(prefilter_kernel<VSAG_AMD_KIND_FP32>, grid, dim3(256), 0, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    return launch_rescore(s, a, nq, k, S, bound, cand, cand_cnt, cap, 0, 0, partial, partial_cnt, nslots, first_slot,
                          out_slot, gate, st);
}

}  // namespace vsag_amd
