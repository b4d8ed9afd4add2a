// Distances between queries and codes named by inner id (FlattenDataCell::Query, src/datacell/flatten_datacell.h:334-440;
// BucketDataCell::QueryOneById, src/datacell/bucket_datacell.h:353-383 -- what Index::CalDistanceById and a reorder
// over quantised codes are made of), and the residual helpers of BucketDataCell (bucket_datacell.h:527-572,594-639).
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

uint64_t rabitq_query_code_size(uint32_t dim, int metric, int query_bits);
int prepare_queries(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, const QueryLayout& ql,
                    uint32_t* qtab, float* qmeta, uint8_t* qcodes, hipStream_t st);
ScanArgs make_scan_args(const vsag_amd_store* s, const QueryLayout& ql, const uint32_t* qtab, const float* qmeta);

struct LookupArgs {
    const uint32_t* ids;         // nq x count inner ids, VSAG_AMD_INVALID_ID = no code
    uint32_t count;
    uint64_t n;                  // codes in the store
    const uint32_t* slot_of_id;  // posting-list stores; null: slot = id
    float* dists;                // nq x count; -1 where there is no code
    // residual stores
    const float* queries;        // raw queries, nq x dim
    const float* bias;           // per slot (l2), or null
    const float* centroids;      // nlist x dim, or null: no residual
    const uint32_t* list_tile;   // 2 nlist
    uint32_t nlist;
    int metric;
};

__global__ void
fill_dists_kernel(float* p, uint64_t n, float v) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// <q, c> and <q, q> summed by one lane in the order a wave sums them in residual_terms_kernel (lane l takes the
// dimensions l, l + 64, ...; the lanes are then added pairwise at distances 32, 16, ... 1), so that a distance looked
// up by id is bit for bit the distance a scan of the list reports.
__device__ inline void
dot_in_wave_order(const float* qv, const float* c, uint32_t dim, float* ip_out, float* qq_out) {
    float ip_stack[7], qq_stack[7];
    int sp = 0;
#pragma unroll
    for (uint32_t j = 0; j < kWave; ++j) {
        // the lane whose partial sum is the j-th leaf of the addition tree: j with its six bits reversed
        const uint32_t leaf = ((j & 1) << 5) | ((j & 2) << 3) | ((j & 4) << 1) | ((j & 8) >> 1) | ((j & 16) >> 3) |
                              ((j & 32) >> 5);
        float ip = 0.0F, qq = 0.0F;
        for (uint32_t d = leaf; d < dim; d += kWave) {
            ip = fmaf(qv[d], c[d], ip);
            qq = fmaf(qv[d], qv[d], qq);
        }
        uint32_t m = j;
        while (m & 1) {
            --sp;
            ip = ip_stack[sp] + ip;
            qq = qq_stack[sp] + qq;
            m >>= 1;
        }
        ip_stack[sp] = ip;
        qq_stack[sp] = qq;
        ++sp;
    }
    *ip_out = ip_stack[0];
    *qq_out = qq_stack[0];
}

// One wave per (query, 64 ids): every lane gathers the granules of its own code.
template <int KIND, int METRIC>
__global__ void __launch_bounds__(64)
store_distances_kernel(ScanArgs a, LookupArgs p) {
    const uint32_t lane = threadIdx.x;
    const uint32_t q = blockIdx.y;
    const uint32_t i = blockIdx.x * kWave + lane;
    const bool have = i < p.count;
    const uint32_t id = have ? p.ids[static_cast<uint64_t>(q) * p.count + i] : VSAG_AMD_INVALID_ID;
    const bool real = id != VSAG_AMD_INVALID_ID && id < p.n;
    const uint32_t slot = real ? (p.slot_of_id != nullptr ? p.slot_of_id[id] : id) : 0U;
    const uint64_t tile = slot >> 6;
    const uint32_t ln = slot & 63;
    const uint32_t qidx[1] = {q};
    const QueryRows<1> qrows = query_rows<1>(a, qidx);
    Acc<KIND, 1> acc;
    acc_reset(acc);
    for (uint32_t j = 0; j < a.G; ++j) {
        const uint4 c = a.tiles[(tile * a.G + j) * kWave + ln];
        accumulate_granule<KIND, METRIC, 1>(a, qrows, j, c, acc);
    }
    float d[1];
    finish_distances<KIND, METRIC, 1>(a, qidx, slot, acc, d);
    float out = d[0];
    if (p.centroids != nullptr && real) {
        // the list of the slot: the last one whose first tile is at or before it
        uint32_t lo = 0, hi = p.nlist;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (p.list_tile[2 * mid] <= tile) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        const float* c = p.centroids + static_cast<uint64_t>(lo) * a.dim;
        const float* qv = p.queries + static_cast<uint64_t>(q) * a.dim;
        float ip, qq;
        dot_in_wave_order(qv, c, a.dim, &ip, &qq);
        if (p.metric == VSAG_AMD_METRIC_COSINE) {
            const float norm = sqrtf(qq);
            ip = ip / (norm == 0.0F ? 1.0F : norm);
        }
        if (p.metric == VSAG_AMD_METRIC_L2) {
            out = (out - (p.bias != nullptr ? p.bias[slot] : 0.0F)) - 2.0F * ip;
        } else {
            out = out - ip;
        }
    }
    if (have) {
        p.dists[static_cast<uint64_t>(q) * p.count + i] = real ? out : -1.0F;
    }
}

template <int KIND>
static void
launch_lookup_m(int metric, dim3 grid, hipStream_t st, const ScanArgs& a, const LookupArgs& p) {
    if (metric == VSAG_AMD_METRIC_L2) {
        hipLaunchKernelGGL((store_distances_kernel<KIND, VSAG_AMD_METRIC_L2>), grid, dim3(kWave), 0, st, a, p);
    } else if (metric == VSAG_AMD_METRIC_COSINE && (KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32)) {
        hipLaunchKernelGGL((store_distances_kernel<KIND, VSAG_AMD_METRIC_COSINE>), grid, dim3(kWave), 0, st, a, p);
    } else {
        hipLaunchKernelGGL((store_distances_kernel<KIND, VSAG_AMD_METRIC_IP>), grid, dim3(kWave), 0, st, a, p);
    }
}

struct LookupBuffers {
    uint32_t* qtab;
    float* qmeta;
    uint8_t* qcodes;
};

static size_t
carve_lookup(Carver& c, const vsag_amd_store* s, uint64_t nq, LookupBuffers* b) {
    const QueryLayout ql = query_layout(s);
    size_t qcode_bytes = query_staging_bytes(s, nq);
    b->qtab = c.take<uint32_t>(nq * ql.qstride);
    b->qmeta = c.take<float>(nq * ql.qmeta);
    b->qcodes = c.take<uint8_t>(qcode_bytes);
    return c.used;
}

// x_i (normalised for cosine) minus the centroid of its list (BucketDataCell::Train / encode_vector,
// bucket_datacell.h:594-625).
__global__ void __launch_bounds__(256)
residual_rows_kernel(const float* x, uint64_t n, uint32_t dim, int metric, const int32_t* labels, const float* centroids,
                     float* out) {
    __shared__ float red[4];
    const uint64_t row = blockIdx.x;
    const float* src = x + row * dim;
    const float* c = centroids + static_cast<uint64_t>(labels[row]) * dim;
    float norm = 1.0F;
    if (metric == VSAG_AMD_METRIC_COSINE) {
        // Normalize (src/simd/generic.cpp:874-878): sqrt of the sequential sum, a zero norm divides by 1
        float s = 0.0F;
        if (threadIdx.x == 0) {
            for (uint32_t d = 0; d < dim; ++d) {
                s = src[d] * src[d] + s;
            }
            red[0] = sqrtf(s);
        }
        __syncthreads();
        norm = red[0] == 0.0F ? 1.0F : red[0];
    }
    for (uint32_t d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = metric == VSAG_AMD_METRIC_COSINE ? src[d] / norm : src[d];
        out[row * dim + d] = v - c[d];
    }
}

// -2 <c, v> - <c, c> for the decoded vectors v (encode_vector, bucket_datacell.h:626-636), one thread per row, sums in
// element order.
__global__ void __launch_bounds__(256)
residual_bias_kernel(const float* decoded, uint64_t n, uint32_t dim, const int32_t* labels, const float* centroids,
                     float* bias) {
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (row >= n) {
        return;
    }
    const float* v = decoded + row * dim;
    const float* c = centroids + static_cast<uint64_t>(labels[row]) * dim;
    float cv = 0.0F, cc = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        cv = c[d] * v[d] + cv;
        cc = c[d] * c[d] + cc;
    }
    bias[row] = -2.0F * cv - cc;
}

// DecodeOneImpl of the scalar quantizers (scalar_quantizer.cpp:114-121, sq8_uniform_quantizer.cpp:140-145,
// sq4_uniform_quantizer.cpp:160-170) and of fp32 (a copy).
__global__ void __launch_bounds__(256)
decode_kernel(int kind, const uint8_t* codes, uint64_t n, uint32_t dim, uint32_t code_size, const float* lb,
              const float* diff, float ulb, float udiff, float* out) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n * dim) {
        return;
    }
    const uint64_t row = i / dim;
    const uint32_t d = static_cast<uint32_t>(i % dim);
    const uint8_t* c = codes + row * code_size;
    float v = 0.0F;
    switch (kind) {
        case VSAG_AMD_KIND_FP32:
            v = reinterpret_cast<const float*>(c)[d];
            break;
        case VSAG_AMD_KIND_SQ8:
            v = static_cast<float>(c[d]) / 255.0F * diff[d] + lb[d];
            break;
        case VSAG_AMD_KIND_SQ4:
            v = static_cast<float>((c[d >> 1] >> (4 * (d & 1))) & 15) / 15.0F * diff[d] + lb[d];
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            v = static_cast<float>(static_cast<double>(c[d]) / 255.0 * static_cast<double>(udiff) + static_cast<double>(ulb));
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            v = static_cast<float>(static_cast<double>((c[d >> 1] >> (4 * (d & 1))) & 15) / 15.0 * static_cast<double>(udiff) +
                                   static_cast<double>(ulb));
            break;
        default:
            break;
    }
    out[i] = v;
}

// Per (query, probed list): <q, c> (twice that for l2), what ScanBucketById takes off every distance of the list
// (bucket_datacell.h:553-566).  One wave per pair.
__global__ void __launch_bounds__(64)
residual_terms_kernel(const float* queries, uint64_t nq, uint32_t dim, int metric, const float* centroids, uint32_t nlist,
                      const int32_t* buckets, uint32_t nprobe, float* terms) {
    const uint64_t pair = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint64_t q = pair / nprobe;
    const int32_t b = buckets[pair];
    if (b < 0 || static_cast<uint32_t>(b) >= nlist) {
        if (lane == 0) {
            terms[pair] = 0.0F;
        }
        return;
    }
    const float* qv = queries + q * dim;
    const float* c = centroids + static_cast<uint64_t>(b) * dim;
    float ip = 0.0F, qq = 0.0F;
    for (uint32_t d = lane; d < dim; d += kWave) {
        ip = fmaf(qv[d], c[d], ip);
        qq = fmaf(qv[d], qv[d], qq);
    }
    for (int off = 32; off > 0; off >>= 1) {
        ip += __shfl_xor(ip, off);
        qq += __shfl_xor(qq, off);
    }
    if (lane == 0) {
        if (metric == VSAG_AMD_METRIC_COSINE) {
            const float norm = sqrtf(qq);
            ip = ip / (norm == 0.0F ? 1.0F : norm);
        }
        terms[pair] = metric == VSAG_AMD_METRIC_L2 ? 2.0F * ip : ip;
    }
}

int
launch_residual_terms(const vsag_amd_store* s, const float* queries, uint64_t nq, const int32_t* buckets, uint32_t nprobe,
                      float* terms, hipStream_t st) {
    hipLaunchKernelGGL(residual_terms_kernel, dim3(static_cast<uint32_t>(nq * nprobe)), dim3(kWave), 0, st, queries, nq,
                       s->dim, s->metric, s->residual_centroids_dev, s->nlist, buckets, nprobe, terms);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_store_distances_workspace_bytes(const vsag_amd_store_t* s, uint64_t nq) {
    if (s == nullptr || nq == 0) {
        return 0;
    }
    Carver c(nullptr, 0);
    LookupBuffers b;
    return carve_lookup(c, s, nq, &b) + 256;
}

extern "C" int
vsag_amd_store_distances(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, const uint32_t* ids_dev,
                         uint32_t count, float* dists_dev, void* workspace_dev, size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(nq >= 1 && nq <= 65535, "nq must be in [1, 65535], got %llu", static_cast<unsigned long long>(nq));
    VA_CHECK_ARG(count >= 1, "count must be positive");
    VA_CHECK_ARG(queries_dev && ids_dev && dists_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver c(workspace_dev, workspace_bytes);
    LookupBuffers b;
    carve_lookup(c, s, nq, &b);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    const QueryLayout ql = query_layout(s);
    VA_TRY(prepare_queries(s, queries_dev, nq, nq, ql, b.qtab, b.qmeta, b.qcodes, st));
    ScanArgs a = make_scan_args(s, ql, b.qtab, b.qmeta);
    LookupArgs p{};
    p.ids = ids_dev;
    p.count = count;
    p.n = s->n;
    p.slot_of_id = s->nlist > 0 ? s->slot_of_id_dev : nullptr;
    p.dists = dists_dev;
    p.queries = queries_dev;
    p.bias = s->residual_bias_dev;
    p.centroids = s->nlist > 0 ? s->residual_centroids_dev : nullptr;
    p.list_tile = s->list_tile_dev;
    p.nlist = s->nlist;
    p.metric = s->metric;
    if (s->n == 0) {
        // an empty store knows no id
        hipLaunchKernelGGL(fill_dists_kernel, dim3(static_cast<uint32_t>(div_up(nq * count, 256))), dim3(256), 0, st,
                           dists_dev, nq * count, -1.0F);
        VA_HIP(hipGetLastError());
        return 0;
    }
    dim3 grid(static_cast<uint32_t>(div_up(count, kWave)), static_cast<uint32_t>(nq));
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
            launch_lookup_m<VSAG_AMD_KIND_FP32>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_SQ8:
            launch_lookup_m<VSAG_AMD_KIND_SQ8>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_SQ4:
            launch_lookup_m<VSAG_AMD_KIND_SQ4>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            launch_lookup_m<VSAG_AMD_KIND_SQ4_UNIFORM>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            launch_lookup_m<VSAG_AMD_KIND_SQ8_UNIFORM>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_PQFS:
            launch_lookup_m<VSAG_AMD_KIND_PQFS>(s->metric, grid, st, a, p);
            break;
        case VSAG_AMD_KIND_RABITQ:
            if (s->query_bits == 32) {
                launch_lookup_m<kKindRabitqF32>(s->metric, grid, st, a, p);
            } else {
                launch_lookup_m<VSAG_AMD_KIND_RABITQ>(s->metric, grid, st, a, p);
            }
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_residual_rows(const float* x_dev, uint64_t n, uint32_t dim, int metric, const int32_t* labels_dev,
                       const float* centroids_dev, float* out_dev, void* stream) {
    VA_TRY(ensure_init());
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(x_dev && labels_dev && centroids_dev && out_dev, "null pointer");
    VA_CHECK_ARG(n < (1ull << 31), "n must be below 2^31");
    hipLaunchKernelGGL(residual_rows_kernel, dim3(static_cast<uint32_t>(n)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       x_dev, n, dim, metric, labels_dev, centroids_dev, out_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_residual_bias(const vsag_amd_store_t* s, const uint8_t* codes_dev, uint64_t n, const int32_t* labels_dev,
                       const float* centroids_dev, float* bias_dev, float* decoded_dev, void* stream) {
    VA_TRY(ensure_init());
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(s && codes_dev && labels_dev && centroids_dev && bias_dev && decoded_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->kind == VSAG_AMD_KIND_RABITQ) {
        if (s->base_bits == 1) {
            VA_TRY(vsag_amd_rabitq_decode(codes_dev, n, s->dim, s->rotation_dev, s->centroid_dev, s->metric,
                                          rabitq_bits_word(s), decoded_dev, stream));
        } else {
            // RaBitQuantizer::DecodeOneImpl returns false for multi-bit codes and writes nothing: encode_vector
            // (bucket_datacell.h:645-650) then takes the products with its zero-initialised buffer.
            VA_HIP(hipMemsetAsync(decoded_dev, 0, n * s->dim * sizeof(float), st));
        }
    } else if (s->kind == VSAG_AMD_KIND_PQFS) {
        VA_TRY(vsag_amd_pq_decode(codes_dev, n, s->dim, s->pq_dim, s->codebooks_dev, decoded_dev, stream));
    } else {
        hipLaunchKernelGGL(decode_kernel, dim3(static_cast<uint32_t>(div_up(n * s->dim, 256))), dim3(256), 0, st, s->kind,
                           codes_dev, n, s->dim, s->code_size, s->lb_dev, s->diff_dev, s->ulb, s->udiff, decoded_dev);
    }
    hipLaunchKernelGGL(residual_bias_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, decoded_dev, n,
                       s->dim, labels_dev, centroids_dev, bias_dev);
    VA_HIP(hipGetLastError());
    return 0;
}
