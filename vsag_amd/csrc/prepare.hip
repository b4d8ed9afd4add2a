// Query preparation for the scans: ProcessQueryImpl of every store kind, written into the tables the
// distance loops read through scalar loads (one row per query, rows aligned to 64 bytes).
#include "distance.h"
#include "store.h"

namespace vsag_amd {

// ------------------------------------------------------------------ query preparation
// One workgroup (256 threads) per query row; rows >= nq are written as zeros so that a partly filled
// query tile computes harmless values.
__device__ inline float
block_sum(float v, float* red) {
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_down(v, off);
    }
    uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        red[wave] = v;
    }
    __syncthreads();
    float s = 0;
    for (uint32_t i = 0; i < (blockDim.x >> 6); ++i) {
        s += red[i];
    }
    __syncthreads();
    return s;
}

// fp32 / sq8 / sq4 tables (ProcessQueryImpl of fp32_quantizer.cpp:216-233 and scalar_quantizer.cpp:154-171
// keep the query in fp32, normalised for cosine; the per-dimension constants are folded in here).
__global__ void __launch_bounds__(256)
prepare_float_queries(const float* q, uint64_t nq, uint32_t dim, int kind, int metric, const float* scale,
                      const float* lb, float* qtab, uint32_t qstride, float* qmeta, uint32_t qmeta_stride) {
    __shared__ float red[4];
    uint64_t row = blockIdx.x;
    float* out = qtab + row * qstride;
    if (row >= nq) {
        for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
            out[d] = 0.0F;
        }
        if (threadIdx.x < qmeta_stride) {
            qmeta[row * qmeta_stride + threadIdx.x] = 0.0F;
        }
        return;
    }
    const float* src = q + row * dim;
    float inv_norm = 1.0F;
    bool cosine = metric == VSAG_AMD_METRIC_COSINE;
    if (cosine) {
        float s = 0;
        for (uint32_t d = threadIdx.x; d < dim; d += blockDim.x) {
            s += src[d] * src[d];
        }
        s = block_sum(s, red);
        inv_norm = sqrtf(s);
        if (inv_norm == 0.0F) {
            inv_norm = 1.0F;  // DivScalarImpl (src/simd/kernels/scalar_op.h:40-42): a zero norm divides by 1
        }
    }
    float bias = 0;
    for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
        float v = 0.0F;
        if (d < dim) {
            float x = cosine ? src[d] / inv_norm : src[d];
            if (kind == VSAG_AMD_KIND_FP32) {
                v = x;
            } else if (metric == VSAG_AMD_METRIC_L2) {
                v = x - lb[d];
            } else {
                v = x * scale[d];
                bias += x * lb[d];
            }
        }
        out[d] = v;
    }
    if (kind != VSAG_AMD_KIND_FP32 && metric != VSAG_AMD_METRIC_L2) {
        bias = block_sum(bias, red);
        if (threadIdx.x == 0) {
            qmeta[row * qmeta_stride] = bias;
        }
    } else if (threadIdx.x < qmeta_stride) {
        qmeta[row * qmeta_stride + threadIdx.x] = 0.0F;
    }
}

// Uniform kinds: the query has been encoded with the base encoder (ProcessQueryImpl = EncodeOneImpl,
// sq4_uniform_quantizer.cpp:204-215, sq8_uniform_quantizer.cpp:178-190); split it into the dwords the
// scan consumes.  meta_off = byte offset of the query's norm (u64, L2) or sum (f32, IP / cosine).
__global__ void __launch_bounds__(256)
prepare_uniform_queries(const uint8_t* qcodes, uint64_t nq, uint32_t code_size, uint32_t payload, int bits,
                        uint32_t meta_off, int meta_u64, uint32_t ndw, uint32_t* qtab, uint32_t qstride,
                        float* qmeta, uint32_t qmeta_stride) {
    uint64_t row = blockIdx.x;
    uint32_t* out = qtab + row * qstride;
    if (row >= nq) {
        for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
            out[d] = 0;
        }
        if (threadIdx.x < qmeta_stride) {
            qmeta[row * qmeta_stride + threadIdx.x] = 0.0F;
        }
        return;
    }
    const uint8_t* c = qcodes + row * code_size;
    for (uint32_t w = threadIdx.x; w < ndw; w += blockDim.x) {
        uint32_t v = 0;
        for (uint32_t b = 0; b < 4; ++b) {
            uint32_t idx = 4 * w + b;
            if (idx < payload) {
                v |= static_cast<uint32_t>(c[idx]) << (8 * b);
            }
        }
        if (bits == 4) {
            out[2 * w] = v & 0x0F0F0F0FU;
            out[2 * w + 1] = (v >> 4) & 0x0F0F0F0FU;
        } else {
            out[w] = v;
        }
    }
    if (threadIdx.x == 0) {
        float m;
        if (meta_u64) {
            uint64_t nrm = 0;
            for (int b = 0; b < 8; ++b) {
                nrm |= static_cast<uint64_t>(c[meta_off + b]) << (8 * b);
            }
            m = static_cast<float>(nrm);
        } else {
            uint32_t u = 0;
            for (int b = 0; b < 4; ++b) {
                u |= static_cast<uint32_t>(c[meta_off + b]) << (8 * b);
            }
            m = __uint_as_float(u);
        }
        qmeta[row * qmeta_stride] = m;
        for (uint32_t i = 1; i < qmeta_stride; ++i) {
            qmeta[row * qmeta_stride + i] = 0.0F;
        }
    }
}

// RaBitQ: processed queries in the reference layout (four planes aligned_dim/8 bytes apart, then lb,
// delta, code sum, norm, raw norm: rabitq_quantizer.cpp:135-176) -> plane-interleaved dwords + the
// per-query factors of recover_dist_between_sq4u_and_fp32 (rabitq_quantizer.cpp:924-939).
__global__ void __launch_bounds__(256)
prepare_rabitq_queries(const uint8_t* qcodes, uint64_t nq, uint32_t qcode_size, uint32_t plane_bytes, uint32_t dim,
                       int has_raw_norm, uint32_t ndw, uint32_t* qtab, uint32_t qstride, float* qmeta,
                       uint32_t qmeta_stride) {
    uint64_t row = blockIdx.x;
    uint32_t* out = qtab + row * qstride;
    if (row >= nq) {
        for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
            out[d] = 0;
        }
        if (threadIdx.x < qmeta_stride) {
            qmeta[row * qmeta_stride + threadIdx.x] = 0.0F;
        }
        return;
    }
    const uint8_t* c = qcodes + row * qcode_size;
    uint32_t code_bytes = (dim + 7) / 8;
    for (uint32_t i = threadIdx.x; i < ndw * 4; i += blockDim.x) {
        uint32_t w = i >> 2, b = i & 3;
        uint32_t v = 0;
        for (uint32_t k = 0; k < 4; ++k) {
            uint32_t idx = 4 * w + k;
            if (idx < code_bytes) {
                v |= static_cast<uint32_t>(c[b * plane_bytes + idx]) << (8 * k);
            }
        }
        out[i] = v;
    }
    if (threadIdx.x == 0) {
        const uint8_t* tail = c + 4 * static_cast<uint64_t>(plane_bytes);
        auto rd = [&](uint32_t off) {
            uint32_t u = 0;
            for (int b = 0; b < 4; ++b) {
                u |= static_cast<uint32_t>(tail[off + b]) << (8 * b);
            }
            return __uint_as_float(u);
        };
        float lb = rd(0), delta = rd(4), qsum = rd(8), qnorm = rd(12);
        float qraw = has_raw_norm ? rd(16) : 0.0F;
        float inv_sqrt_d = 1.0F / sqrtf(static_cast<float>(dim));
        float* m = qmeta + row * qmeta_stride;
        m[0] = inv_sqrt_d * delta * 2;
        m[1] = inv_sqrt_d * lb * 2;
        m[2] = inv_sqrt_d * delta * qsum;
        m[3] = inv_sqrt_d * lb * static_cast<float>(dim);
        m[4] = qnorm;
        m[5] = qraw;
        m[6] = 0;
        m[7] = 0;
    }
}

uint64_t rabitq_query_code_size(uint32_t dim, int metric, int query_bits);
int squ_encode_launch(const float* x, uint64_t n, uint32_t dim, int bits, int metric, const float* bounds,
                      uint8_t* codes, hipStream_t st, float* norm_scratch);
int rabitq_process_query_launch(const float* q, uint64_t nq, uint32_t dim, const float* rot, const float* centroid,
                                int metric, int query_bits, uint8_t* qcodes, hipStream_t st, float* scratch);

// Bytes of the encoded queries of a call (uniform kinds, rabitq; zero for the kinds that keep fp32 queries).
static size_t
query_code_bytes(const vsag_amd_store* s, uint64_t nq) {
    if (s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
        return nq * s->code_size;
    }
    if (s->kind == VSAG_AMD_KIND_RABITQ) {
        return nq * rabitq_query_code_size(s->dim, s->metric, rabitq_bits_word(s));
    }
    return 0;
}

// What the query encoders need besides their output: the rotated queries of one slab (rabitq), a norm per
// query (uniform kinds under cosine).
static size_t
query_scratch_bytes(const vsag_amd_store* s, uint64_t nq) {
    if (s->kind == VSAG_AMD_KIND_RABITQ) {
        return static_cast<size_t>(nq < kRotateSlabRows ? nq : kRotateSlabRows) * s->dim * 4;
    }
    if ((s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) &&
        s->metric == VSAG_AMD_METRIC_COSINE) {
        return nq * 4;
    }
    return 0;
}

size_t
query_staging_bytes(const vsag_amd_store* s, uint64_t nq) {
    size_t scratch = query_scratch_bytes(s, nq);
    return scratch == 0 ? query_code_bytes(s, nq) : round_up(query_code_bytes(s, nq), 256) + scratch;
}

int pqfs_prepare_launch(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, uint32_t* qtab,
                        uint32_t qstride, float* qmeta, uint32_t qmeta_stride, hipStream_t st);

QueryLayout
query_layout(const vsag_amd_store* s) {
    QueryLayout l{};
    uint32_t ndw = s->G * 4;
    switch (s->kind) {
        case VSAG_AMD_KIND_PQFS:
            l.qstride = s->G * 128;  // 16 table bytes for each of the 32 subspaces of a granule
            l.qmeta = 2;
            break;
        case VSAG_AMD_KIND_FP32:
            l.qstride = s->dpad;
            l.qmeta = 1;
            break;
        case VSAG_AMD_KIND_SQ8:
        case VSAG_AMD_KIND_SQ4:
            l.qstride = s->dpad;
            l.qmeta = 1;
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            l.qstride = ndw * 2;
            l.qmeta = 1;
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            l.qstride = ndw;
            l.qmeta = 1;
            break;
        case VSAG_AMD_KIND_RABITQ:
            l.qstride = s->query_bits == 32 ? s->dpad : ndw * 4;
            l.qmeta = 8;
            break;
    }
    // Rows start on a 64-byte boundary so that scalar dwordx16 loads stay aligned.
    l.qstride = static_cast<uint32_t>(round_up(l.qstride, 16));
    return l;
}

// Processed fp32 queries of a RaBitQ store (the normalised rotated residual, its norm, the raw norm:
// rabitq_quantizer.cpp:2049-2088) -> table row padded with zeros + the factors of the estimator.
__global__ void __launch_bounds__(256)
prepare_rabitq_f32_queries(const uint8_t* qcodes, uint64_t nq, uint32_t qcode_size, uint32_t dim, int has_raw_norm,
                           int has_sum, uint32_t* qtab, uint32_t qstride, float* qmeta, uint32_t qmeta_stride) {
    __shared__ float partial[256];
    uint64_t row = blockIdx.x;
    uint32_t* out = qtab + row * qstride;
    if (row >= nq) {
        for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
            out[d] = 0;
        }
        if (threadIdx.x < qmeta_stride) {
            qmeta[row * qmeta_stride + threadIdx.x] = 0.0F;
        }
        return;
    }
    const uint8_t* c = qcodes + row * qcode_size;
    auto rd = [&](uint32_t off) {
        uint32_t u = 0;
        for (int b = 0; b < 4; ++b) {
            u |= static_cast<uint32_t>(c[off + b]) << (8 * b);
        }
        return u;
    };
    float s = 0.0F;
    for (uint32_t d = threadIdx.x; d < qstride; d += blockDim.x) {
        uint32_t u = d < dim ? rd(4 * d) : 0U;
        out[d] = u;
        s += __uint_as_float(u);
    }
    partial[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.0F;
        for (uint32_t i = 0; i < blockDim.x; ++i) {
            total += partial[i];
        }
        // behind the values: (their running sum, multi-bit base codes only,) the norm, (the raw norm)
        uint32_t tail = (4 * dim + 3) / 4 * 4 + (has_sum ? 4 : 0);
        float inv_sqrt_d = 1.0F / sqrtf(static_cast<float>(dim));
        float* m = qmeta + row * qmeta_stride;
        m[0] = 2.0F * inv_sqrt_d;
        m[1] = has_sum ? __uint_as_float(rd(4 * dim)) : 0.0F;
        m[2] = inv_sqrt_d * total;
        m[3] = 0.0F;
        m[4] = __uint_as_float(rd(tail));
        m[5] = has_raw_norm ? __uint_as_float(rd(tail + 4)) : 0.0F;
    }
}

// Runs ProcessQueryImpl of the store's quantizer for nq raw queries and fills the scan tables.  `qcodes` is
// query_staging_bytes(s, nq) of device memory (the encoded queries, then the encoders' scratch): nothing is
// allocated here.
int
prepare_queries(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, const QueryLayout& ql,
                uint32_t* qtab, float* qmeta, uint8_t* qcodes, hipStream_t st) {
    dim3 grid(static_cast<uint32_t>(nq_pad));
    float* scratch = query_scratch_bytes(s, nq) == 0 ? nullptr :
                     reinterpret_cast<float*>(qcodes + round_up(query_code_bytes(s, nq), 256));
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
        case VSAG_AMD_KIND_SQ8:
        case VSAG_AMD_KIND_SQ4:
            hipLaunchKernelGGL(prepare_float_queries, grid, dim3(256), 0, st, queries, nq, s->dim, s->kind, s->metric,
                               s->scale_dev, s->lb_dev, reinterpret_cast<float*>(qtab), ql.qstride, qmeta, ql.qmeta);
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
        case VSAG_AMD_KIND_SQ8_UNIFORM: {
            int bits = s->kind == VSAG_AMD_KIND_SQ4_UNIFORM ? 4 : 8;
            VA_TRY(squ_encode_launch(queries, nq, s->dim, bits, s->metric, s->bounds_dev, qcodes, st, scratch));
            hipLaunchKernelGGL(prepare_uniform_queries, grid, dim3(256), 0, st, qcodes, nq, s->code_size,
                               s->payload_bytes, bits, s->meta_offset[0], static_cast<int>(s->meta_is_u64 & 1),
                               s->G * 4, qtab, ql.qstride, qmeta, ql.qmeta);
            break;
        }
        case VSAG_AMD_KIND_RABITQ: {
            VA_CHECK_ARG(s->query_bits == 4 || s->query_bits == 32, "rabitq scan supports 4-bit and fp32 queries");
            VA_TRY(rabitq_process_query_launch(queries, nq, s->dim, s->rotation_dev, s->centroid_dev, s->metric,
                                               rabitq_bits_word(s), qcodes, st, scratch));
            if (s->query_bits == 32) {
                hipLaunchKernelGGL(prepare_rabitq_f32_queries, grid, dim3(256), 0, st, qcodes, nq,
                                   static_cast<uint32_t>(rabitq_query_code_size(s->dim, s->metric, rabitq_bits_word(s))),
                                   s->dim, s->metric != VSAG_AMD_METRIC_L2 ? 1 : 0, s->base_bits != 1 ? 1 : 0, qtab,
                                   ql.qstride, qmeta, ql.qmeta);
                break;
            }
            uint32_t aligned_dim = (s->dim + 511) / 512 * 512;
            hipLaunchKernelGGL(prepare_rabitq_queries, grid, dim3(256), 0, st, qcodes, nq,
                               static_cast<uint32_t>(rabitq_query_code_size(s->dim, s->metric, s->query_bits)),
                               aligned_dim / 8, s->dim, s->metric != VSAG_AMD_METRIC_L2 ? 1 : 0, s->G * 4, qtab,
                               ql.qstride, qmeta, ql.qmeta);
            break;
        }
        case VSAG_AMD_KIND_PQFS:
            VA_TRY(pqfs_prepare_launch(s, queries, nq, nq_pad, qtab, ql.qstride, qmeta, ql.qmeta, st));
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

ScanArgs
make_scan_args(const vsag_amd_store* s, const QueryLayout& ql, const uint32_t* qtab, const float* qmeta) {
    ScanArgs a{};
    a.tiles = s->tiles;
    a.meta = s->meta;
    a.meta_stride = s->cap_tiles * kWave;
    a.scale = s->scale_dev;
    a.qtab = qtab;
    a.qmeta = qmeta;
    a.qstride = ql.qstride;
    a.qmeta_stride = ql.qmeta;
    a.G = s->G;
    a.dim = s->dim;
    a.planes = s->planes;
    a.plane_granules = s->plane_granules;
    a.plane_recip = (65536U + s->plane_granules - 1) / s->plane_granules;
    a.f0 = s->ulb;
    a.f1 = s->scalar_rate;
    a.f2 = s->ulb * s->ulb;
    return a;
}
}  // namespace vsag_amd
