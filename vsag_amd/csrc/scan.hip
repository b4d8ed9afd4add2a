// Flat scan with fused per-query top-k (BruteForce::SearchWithRequest hot loop,
// src/algorithm/bruteforce/bruteforce.cpp:481-597), batched over queries.
//
// Grid: x = query tile (T queries), y = chunk of code tiles.  A workgroup has up to four waves; wave w
// walks tiles chunk_begin + w, + W, ... and keeps one LDS selector per query of the tile.  Workgroups
// that are resident together have consecutive x and the same y, so they stream the same chunk of codes
// at the same time and share it through each XCD's L2.  Every wave leaves its k best keys in a partial
// buffer; a second kernel merges the partials of a query.
#include "distance.h"
#include "store.h"
#include "topk.h"

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

__global__ void
fill_words_kernel(uint32_t* p, uint32_t v, uint64_t n) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// ------------------------------------------------------------------ flat scan
struct FlatArgs {
    uint64_t n;
    uint64_t ntiles;
    uint64_t tiles_per_chunk;
    uint64_t nq;
    uint32_t k;
    uint32_t S;
    uint32_t nslots;   // partial lists per query = chunks * waves
    uint64_t* partial; // nq x nslots x k keys
};

template <int KIND, int METRIC, int T>
__global__ void __launch_bounds__(256)
flat_scan_kernel(ScanArgs a, FlatArgs f) {
    extern __shared__ uint64_t lds[];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nwaves = blockDim.x >> 6;
    const uint32_t S = f.S, k = f.k;
    uint64_t* sel = lds + static_cast<size_t>(wave) * T * S;

    uint32_t qidx[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        qidx[t] = blockIdx.x * T + t;
    }
    for (uint32_t i = lane; i < T * S; i += kWave) {
        sel[i] = kInfKey;
    }
    wave_lds_fence();

    uint32_t cnt[T];
    float tau[T];
    bool open[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        cnt[t] = 0;
        tau[t] = __builtin_inff();
        open[t] = true;
    }

    const uint64_t tile_begin = static_cast<uint64_t>(blockIdx.y) * f.tiles_per_chunk;
    uint64_t tile_end = tile_begin + f.tiles_per_chunk;
    if (tile_end > f.ntiles) {
        tile_end = f.ntiles;
    }
    for (uint64_t tile = tile_begin + wave; tile < tile_end; tile += nwaves) {
        float d[T];
        tile_distances<KIND, METRIC, T>(a, tile, qidx, lane, d);
        const uint64_t id = tile * kWave + lane;
        const bool valid = id < f.n;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            // Inner ids grow along the scan, so `d < tau` is the (distance, id) order exactly.
            bool pass = valid && (open[t] || d[t] < tau[t]);
            uint64_t* keys = sel + t * S;
            cnt[t] = selector_append(keys, k, cnt[t], pass, make_key(d[t], static_cast<uint32_t>(id)));
            if (cnt[t] + kWave > S - k) {
                uint64_t th = selector_flush(keys, S, k, cnt[t], lane);
                cnt[t] = 0;
                open[t] = th == kInfKey;
                tau[t] = open[t] ? __builtin_inff() : ordered_to_float(static_cast<uint32_t>(th >> 32));
            }
        }
    }
    const uint32_t slot = blockIdx.y * nwaves + wave;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        uint64_t* keys = sel + t * S;
        selector_flush(keys, S, k, cnt[t], lane);
        if (qidx[t] < f.nq) {
            uint64_t* dst = f.partial + (static_cast<uint64_t>(qidx[t]) * f.nslots + slot) * k;
            for (uint32_t i = lane; i < k; i += kWave) {
                dst[i] = keys[i];
            }
        }
    }
}

// One wave per query: k best keys of `count` partial keys, written as ids / distances (ascending).
__global__ void __launch_bounds__(64)
merge_partials_kernel(const uint64_t* partial, uint64_t per_query, uint32_t k, uint32_t S, uint32_t* ids,
                      float* dists) {
    extern __shared__ uint64_t lds[];
    const uint32_t lane = threadIdx.x;
    const uint64_t q = blockIdx.x;
    selector_init(lds, S, lane);
    const uint64_t* src = partial + q * per_query;
    uint32_t cnt = 0;
    uint64_t tau = kInfKey;
    for (uint64_t base = 0; base < per_query; base += kWave) {
        uint64_t idx = base + lane;
        uint64_t key = idx < per_query ? src[idx] : kInfKey;
        bool pass = key < tau;
        cnt = selector_append(lds, k, cnt, pass, key);
        if (cnt + kWave > S - k) {
            tau = selector_flush(lds, S, k, cnt, lane);
            cnt = 0;
        }
    }
    selector_flush(lds, S, k, cnt, lane);
    for (uint32_t i = lane; i < k; i += kWave) {
        uint64_t key = lds[i];
        if (key == kInfKey) {
            ids[q * k + i] = VSAG_AMD_INVALID_ID;
            dists[q * k + i] = __builtin_inff();
        } else {
            ids[q * k + i] = static_cast<uint32_t>(key);
            dists[q * k + i] = ordered_to_float(static_cast<uint32_t>(key >> 32));
        }
    }
}

// ------------------------------------------------------------------ host side
static int g_tile_override = 0;
static int g_chunk_override = 0;
static thread_local int tl_last_tile = 0;
static thread_local uint64_t tl_last_passes = 0;
static thread_local uint64_t tl_last_bytes = 0;

QueryLayout
query_layout(const vsag_amd_store* s) {
    QueryLayout l{};
    uint32_t ndw = s->G * 4;
    switch (s->kind) {
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
            l.qstride = ndw * 4;
            l.qmeta = 8;
            break;
    }
    // Rows start on a 64-byte boundary so that scalar dwordx16 loads stay aligned.
    l.qstride = static_cast<uint32_t>(round_up(l.qstride, 16));
    return l;
}

// Largest query tile the kind supports without spilling SGPRs / registers.
static int
default_query_tile(const vsag_amd_store* s, uint64_t nq) {
    int t;
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
            t = 4;
            break;
        case VSAG_AMD_KIND_SQ8:
        case VSAG_AMD_KIND_SQ4:
            t = s->metric == VSAG_AMD_METRIC_L2 ? 2 : 4;
            break;
        case VSAG_AMD_KIND_RABITQ:
            t = 2;
            break;
        default:
            t = 4;
    }
    while (t > 1 && static_cast<uint64_t>(t) > nq) {
        t >>= 1;
    }
    return t;
}

struct ScanPlan {
    int T;
    uint32_t S;
    uint32_t waves;
    uint64_t nq_pad;
    uint64_t chunks;
    uint64_t tiles_per_chunk;
    uint32_t nslots;
    QueryLayout ql;
    size_t qcode_bytes;  // staging for encoded queries (uniform kinds, rabitq)
};

uint64_t rabitq_query_code_size(uint32_t dim, int metric, int query_bits);

static int
make_plan(const vsag_amd_store* s, uint64_t nq, uint32_t k, uint64_t ntiles, ScanPlan* p) {
    p->T = g_tile_override > 0 ? g_tile_override : default_query_tile(s, nq);
    p->S = selector_slots(k);
    // Selectors of one workgroup must fit 64 KiB of LDS.
    while (p->T > 1 && static_cast<size_t>(p->T) * p->S * 8 > 65536) {
        p->T >>= 1;
    }
    uint32_t waves = 4;
    while (waves > 1 && static_cast<size_t>(waves) * p->T * p->S * 8 > 65536) {
        waves >>= 1;
    }
    p->waves = waves;
    p->nq_pad = round_up(nq, p->T);
    uint64_t qtiles = p->nq_pad / p->T;
    uint64_t chunks;
    if (g_chunk_override > 0) {
        chunks = g_chunk_override;
    } else {
        // Enough workgroups for about eight rounds over the machine, but at least 16 tiles per wave.
        uint64_t target = static_cast<uint64_t>(device_cu_count()) * 8 * 8;
        chunks = div_up(target, qtiles);
    }
    uint64_t max_chunks = ntiles / (16 * waves);
    if (max_chunks < 1) {
        max_chunks = 1;
    }
    if (chunks > max_chunks) {
        chunks = max_chunks;
    }
    if (chunks < 1) {
        chunks = 1;
    }
    if (chunks > 65535) {
        chunks = 65535;
    }
    p->tiles_per_chunk = div_up(ntiles > 0 ? ntiles : 1, chunks);
    p->chunks = div_up(ntiles > 0 ? ntiles : 1, p->tiles_per_chunk);
    p->nslots = static_cast<uint32_t>(p->chunks * waves);
    p->ql = query_layout(s);
    p->qcode_bytes = 0;
    if (s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
        p->qcode_bytes = nq * s->code_size;
    } else if (s->kind == VSAG_AMD_KIND_RABITQ) {
        p->qcode_bytes = nq * rabitq_query_code_size(s->dim, s->metric, s->query_bits);
    }
    return 0;
}

struct ScanBuffers {
    uint32_t* qtab;
    float* qmeta;
    uint8_t* qcodes;
    uint64_t* partial;
};

static size_t
carve_scan(Carver& c, const ScanPlan& p, uint64_t partial_keys, ScanBuffers* b) {
    b->qtab = c.take<uint32_t>(p.nq_pad * p.ql.qstride);
    b->qmeta = c.take<float>(p.nq_pad * p.ql.qmeta);
    b->qcodes = c.take<uint8_t>(p.qcode_bytes);
    b->partial = c.take<uint64_t>(partial_keys);
    return c.used;
}

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);
int squ_encode_launch(const float* x, uint64_t n, uint32_t dim, int bits, int metric, const float* bounds,
                      uint8_t* codes, hipStream_t st);
int rabitq_process_query_launch(const float* q, uint64_t nq, uint32_t dim, const float* rot, const float* centroid,
                                int metric, int query_bits, uint8_t* qcodes, hipStream_t st);

// Runs ProcessQueryImpl of the store's quantizer for nq raw queries and fills the scan tables.
int
prepare_queries(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, const QueryLayout& ql,
                uint32_t* qtab, float* qmeta, uint8_t* qcodes, hipStream_t st) {
    dim3 grid(static_cast<uint32_t>(nq_pad));
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
            VA_TRY(squ_encode_launch(queries, nq, s->dim, bits, s->metric, s->bounds_dev, qcodes, st));
            hipLaunchKernelGGL(prepare_uniform_queries, grid, dim3(256), 0, st, qcodes, nq, s->code_size,
                               s->payload_bytes, bits, s->meta_offset[0], static_cast<int>(s->meta_is_u64 & 1),
                               s->G * 4, qtab, ql.qstride, qmeta, ql.qmeta);
            break;
        }
        case VSAG_AMD_KIND_RABITQ: {
            VA_CHECK_ARG(s->query_bits == 4, "rabitq scan supports 4-bit queries only");
            VA_TRY(rabitq_process_query_launch(queries, nq, s->dim, s->rotation_dev, s->centroid_dev, s->metric,
                                               s->query_bits, qcodes, st));
            uint32_t aligned_dim = (s->dim + 511) / 512 * 512;
            hipLaunchKernelGGL(prepare_rabitq_queries, grid, dim3(256), 0, st, qcodes, nq,
                               static_cast<uint32_t>(rabitq_query_code_size(s->dim, s->metric, s->query_bits)),
                               aligned_dim / 8, s->dim, s->metric != VSAG_AMD_METRIC_L2 ? 1 : 0, s->G * 4, qtab,
                               ql.qstride, qmeta, ql.qmeta);
            break;
        }
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
    a.f0 = s->ulb;
    a.f1 = s->scalar_rate;
    a.f2 = s->ulb * s->ulb;
    return a;
}

template <int KIND, int METRIC>
static void
launch_flat_t(int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a, const FlatArgs& f) {
    switch (T) {
        case 1:
            hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, 1>), grid, block, lds, st, a, f);
            break;
        case 2:
            hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, 2>), grid, block, lds, st, a, f);
            break;
        case 4:
            hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, 4>), grid, block, lds, st, a, f);
            break;
        default:
            hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, 8>), grid, block, lds, st, a, f);
            break;
    }
}

template <int KIND>
static void
launch_flat_m(int metric, int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a,
              const FlatArgs& f) {
    // Cosine stores hold normalised vectors and scan as inner product (RaBitQ has its own formula).
    if (metric == VSAG_AMD_METRIC_L2) {
        launch_flat_t<KIND, VSAG_AMD_METRIC_L2>(T, grid, block, lds, st, a, f);
    } else if (metric == VSAG_AMD_METRIC_COSINE && KIND == VSAG_AMD_KIND_RABITQ) {
        launch_flat_t<KIND, VSAG_AMD_METRIC_COSINE>(T, grid, block, lds, st, a, f);
    } else {
        launch_flat_t<KIND, VSAG_AMD_METRIC_IP>(T, grid, block, lds, st, a, f);
    }
}

static int
launch_flat(const vsag_amd_store* s, const ScanPlan& p, const ScanArgs& a, const FlatArgs& f, hipStream_t st) {
    dim3 grid(static_cast<uint32_t>(p.nq_pad / p.T), static_cast<uint32_t>(p.chunks));
    dim3 block(p.waves * kWave);
    size_t lds = static_cast<size_t>(p.waves) * p.T * p.S * 8;
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
            launch_flat_m<VSAG_AMD_KIND_FP32>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_SQ8:
            launch_flat_m<VSAG_AMD_KIND_SQ8>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_SQ4:
            launch_flat_m<VSAG_AMD_KIND_SQ4>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            launch_flat_m<VSAG_AMD_KIND_SQ4_UNIFORM>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            launch_flat_m<VSAG_AMD_KIND_SQ8_UNIFORM>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_RABITQ:
            launch_flat_m<VSAG_AMD_KIND_RABITQ>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

static int
check_scan_call(const vsag_amd_store* s, uint64_t nq, uint32_t k) {
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(k >= 1 && k <= kMaxTopK, "k must be in [1, %u], got %u", kMaxTopK, k);
    VA_CHECK_ARG(nq >= 1 && nq <= (1ull << 31), "nq must be in [1, 2^31], got %llu",
                 static_cast<unsigned long long>(nq));
    return 0;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_flat_scan_workspace_bytes(const vsag_amd_store_t* s, uint64_t nq, uint32_t k) {
    if (check_scan_call(s, nq, k) != 0 || ensure_init() != 0) {
        return 0;
    }
    ScanPlan p;
    make_plan(s, nq, k, s->ntiles, &p);
    Carver c(nullptr, 0);
    ScanBuffers b;
    return carve_scan(c, p, nq * p.nslots * k, &b) + 256;
}

extern "C" int
vsag_amd_flat_scan_topk(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
                        uint32_t* ids_dev, float* dists_dev, void* workspace_dev, size_t workspace_bytes,
                        void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_scan_call(s, nq, k));
    VA_CHECK_ARG(s->nlist == 0, "flat scan on a posting-list store");
    VA_CHECK_ARG(queries_dev && ids_dev && dists_dev, "null query / output pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    ScanPlan p;
    make_plan(s, nq, k, s->ntiles, &p);
    Carver c(workspace_dev, workspace_bytes);
    ScanBuffers b;
    carve_scan(c, p, nq * p.nslots * k, &b);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);

    VA_TRY(prepare_queries(s, queries_dev, nq, p.nq_pad, p.ql, b.qtab, b.qmeta, b.qcodes, st));
    ScanArgs a = make_scan_args(s, p.ql, b.qtab, b.qmeta);
    FlatArgs f{};
    f.n = s->n;
    f.ntiles = s->ntiles;
    f.tiles_per_chunk = p.tiles_per_chunk;
    f.nq = nq;
    f.k = k;
    f.S = p.S;
    f.nslots = p.nslots;
    f.partial = b.partial;
    if (s->ntiles == 0) {
        // Empty store: every slot of the partial buffer must still read as "no candidate".
        uint64_t words = nq * p.nslots * k * 2;
        hipLaunchKernelGGL(fill_words_kernel, dim3(static_cast<uint32_t>(div_up(words, 256))), dim3(256), 0, st,
                           reinterpret_cast<uint32_t*>(b.partial), 0xFFFFFFFFU, words);
    } else {
        timing_begin(st);
        VA_TRY(launch_flat(s, p, a, f, st));
        timing_end(st);
    }
    hipLaunchKernelGGL(merge_partials_kernel, dim3(static_cast<uint32_t>(nq)), dim3(kWave), p.S * 8, st, b.partial,
                       static_cast<uint64_t>(p.nslots) * k, k, p.S, ids_dev, dists_dev);
    VA_HIP(hipGetLastError());
    tl_last_tile = p.T;
    tl_last_passes = p.nq_pad / p.T;
    tl_last_bytes = s->ntiles * s->G * kWave * kGranule;
    return 0;
}

extern "C" int
vsag_amd_set_scan_tuning(int query_tile, int base_chunks) {
    VA_CHECK_ARG(query_tile == 0 || query_tile == 1 || query_tile == 2 || query_tile == 4 || query_tile == 8,
                 "query_tile must be 0, 1, 2, 4 or 8");
    VA_CHECK_ARG(base_chunks >= 0 && base_chunks <= 65535, "base_chunks must be in [0, 65535]");
    g_tile_override = query_tile;
    g_chunk_override = base_chunks;
    return 0;
}

extern "C" int
vsag_amd_last_scan_info(int* query_tile, uint64_t* passes, uint64_t* bytes_per_pass) {
    if (query_tile) {
        *query_tile = tl_last_tile;
    }
    if (passes) {
        *passes = tl_last_passes;
    }
    if (bytes_per_pass) {
        *bytes_per_pass = tl_last_bytes;
    }
    return 0;
}
