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
rabitq_tau_kernel(const float* qmeta, uint32_t qmeta_stride, const uint32_t* bound, int is_l2, uint64_t nq, uint64_t nq_pad,
                  float* u) {
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
                    u4 = static_cast<float>(v4 * lower);
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
};

__device__ inline int
rb_spread(uint32_t nibble) {
    // bit j of the nibble into byte j
    return static_cast<int>((nibble * 0x00204081U) & 0x01010101U);
}

template <int METRIC>
__global__ void __launch_bounds__(kRbThreads, 2)
prefilter_rb_kernel(PrefilterRbArgs p) {
    extern __shared__ uint4 rb_lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint32_t nchunks = 8 * p.G;  // 16-byte chunks per query row: chunk 2 s + h of step s = code dword s
    const uint64_t q0 = static_cast<uint64_t>(blockIdx.y) * kRbQueries;
    uint4* qs = rb_lds;                                                           // [chunk][128 queries]
    float* cc = reinterpret_cast<float*>(rb_lds + nchunks * kRbQueries) + wave * 3 * kWave;  // [3][64] per wave

    // The query group, once: chunk c of query q to qs[c][q].
    for (uint32_t i = tid; i < nchunks * kRbQueries; i += blockDim.x) {
        const uint32_t ql = i / nchunks, c = i % nchunks;
        qs[c * kRbQueries + ql] = p.qbytes[(q0 + ql) * nchunks + c];
    }
    float u1[4], u2[4], u3[4], u4[4];
    uint32_t ncand[4] = {0, 0, 0, 0};
    const uint32_t sub_lists = p.groups * 2 * kRbWaves;
    const uint32_t my_sub = (blockIdx.x * kRbWaves + wave) * 2 + half;
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        const uint64_t q = q0 + 32 * qb + l32;
        u1[qb] = p.u[q];
        u2[qb] = p.u[p.nq_pad + q];
        u3[qb] = p.u[2 * p.nq_pad + q];
        u4[qb] = p.u[3 * p.nq_pad + q];
    }
    __syncthreads();

    const uint64_t span = p.tile_end - p.tile_begin;
    for (uint64_t t = static_cast<uint64_t>(blockIdx.x) * kRbWaves + wave; t < span;
         t += static_cast<uint64_t>(p.groups) * kRbWaves) {
        const uint64_t tile = p.tile_begin + t;
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
        odd = odd || !(a_c <= 64.0F) || !(fabsf(b_c) <= 64.0F) || !(fabsf(bsum) <= 65536.0F);
        a_c = odd ? 0.0F : a_c;
        b_c = odd ? 0.0F : b_c;
        const bool special = odd && my_slot < p.n;
        wave_lds_fence();  // the previous tile's verdicts have read these
        cc[lane] = a_c;
        cc[kWave + lane] = b_c;
        cc[2 * kWave + lane] = odd ? 0.0F : bsum;
        const uint64_t special_mask = __ballot(special);
        wave_lds_fence();

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
                        const uint64_t q = q0 + 32 * qb + l32;
                        uint32_t* list = p.cand + ((q < p.nq ? q : 0) * sub_lists + my_sub) * p.sub_cap;
                        while (hits != 0) {
                            const uint32_t j = static_cast<uint32_t>(__builtin_ctz(hits));
                            hits &= hits - 1;
                            const uint32_t code = row + j;
                            const uint64_t slot = tile * kWave + code;
                            if (slot < p.n && ((special_mask >> code) & 1ULL) == 0) {
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
        // Codes outside the derivation: candidates of every query (lanes of the first half append them).
        if (special_mask != 0 && half == 0) {
            uint64_t rest = special_mask;
            while (rest != 0) {
                const uint32_t code = static_cast<uint32_t>(__builtin_ctzll(rest));
                rest &= rest - 1;
#pragma unroll
                for (int qb = 0; qb < 4; ++qb) {
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
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        const uint64_t q = q0 + 32 * qb + l32;
        if (q < p.nq) {
            p.cand_cnt[q * sub_lists + my_sub] = ncand[qb];
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
                       a.qmeta_stride, bound, l2 ? 1 : 0, nq, nq_pad, u);
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

}  // namespace vsag_amd
