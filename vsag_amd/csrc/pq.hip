// Product quantization in its fast-scan form ("pqfs", src/quantization/product_quantization/pq_fastscan_quantizer.cpp):
// pq_dim subspaces of dim / pq_dim dimensions with 16 centroids each; a code is one 4-bit centroid index per subspace
// (subspace i in byte i / 2, low nibble for even i); a processed query is a table of 16 bytes per subspace -- the
// distances (l2) or inner products (ip, cosine) of its sub-vectors to the centroids, quantised between the smallest
// and largest entry -- plus the two floats that turn a sum of table bytes back into a distance.
//
// Everything order-dependent keeps the element order of the reference's scalar kernels (generic::FP32ComputeL2Sqr,
// generic::Normalize) and is not contracted into fused multiply-adds, so codes, tables and distances equal the CPU
// restatement's bit for bit.  The reference's own ip table comes out of cblas_sgemv, whose order of summation is the
// BLAS library's.
#include <random>
#include <vector>

#include "store.h"

namespace vsag_amd {

constexpr uint32_t kPqCentroids = 16;

// norm[i] = the divisor generic::Normalize uses for row i (src/simd/generic.cpp:874-878: sqrt of the running sum
// x_d x_d + s in element order; a zero norm divides by 1).
__global__ void __launch_bounds__(256)
pq_row_norm_kernel(const float* x, uint64_t n, uint32_t dim, float* norm) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const float* r = x + i * dim;
    float s = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        s = r[d] * r[d] + s;
    }
    const float v = sqrtf(s);
    norm[i] = v == 0.0F ? 1.0F : v;
}

// slice[j][d] = x[j][first + d] (/ norm[j]): the training rows of one subspace (pq_fastscan_quantizer.cpp:80-85).
__global__ void __launch_bounds__(256)
pq_slice_kernel(const float* x, uint64_t n, uint32_t dim, uint32_t first, uint32_t sd, const float* norm, float* slice) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n * sd) {
        return;
    }
    const uint64_t j = i / sd;
    const uint32_t d = static_cast<uint32_t>(i % sd);
    const float v = x[j * dim + first + d];
    slice[i] = norm != nullptr ? v / norm[j] : v;
}

// EncodeOneImpl (pq_fastscan_quantizer.cpp:97-127): a thread per (row, code byte) = two subspaces; per subspace the
// first centroid of smallest squared distance (strict <, from FLT_MAX).
__global__ void __launch_bounds__(256)
pq_encode_kernel(const float* x, uint64_t n, uint32_t dim, uint32_t pq_dim, const float* codebooks, const float* norm,
                 uint8_t* codes, uint32_t code_size) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n * code_size) {
        return;
    }
    const uint64_t row = i / code_size;
    const uint32_t b = static_cast<uint32_t>(i % code_size);
    const uint32_t sd = dim / pq_dim;
    const float scalar = norm != nullptr ? norm[row] : 1.0F;
    uint32_t byte = 0;
    for (uint32_t h = 0; h < 2; ++h) {
        const uint32_t sub = 2 * b + h;
        if (sub >= pq_dim) {
            break;
        }
        const float* q = x + row * dim + static_cast<uint64_t>(sub) * sd;
        const float* base = codebooks + static_cast<uint64_t>(sub) * kPqCentroids * sd;
        float nearest = 3.402823466e+38F;
        uint32_t id = 0;
        for (uint32_t j = 0; j < kPqCentroids; ++j) {
            const float* c = base + static_cast<uint64_t>(j) * sd;
            float s = 0.0F;
            for (uint32_t d = 0; d < sd; ++d) {
                const float v = norm != nullptr ? q[d] / scalar : q[d];
                const float t = v - c[d];
                s = t * t + s;
            }
            if (s < nearest) {
                nearest = s;
                id = j;
            }
        }
        byte |= id << (4 * h);
    }
    codes[i] = static_cast<uint8_t>(byte);
}

// DecodeOneImpl (pq_fastscan_quantizer.cpp:140-156).
__global__ void __launch_bounds__(256)
pq_decode_kernel(const uint8_t* codes, uint64_t n, uint32_t dim, uint32_t pq_dim, const float* codebooks,
                 uint32_t code_size, float* out) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n * dim) {
        return;
    }
    const uint64_t row = i / dim;
    const uint32_t d = static_cast<uint32_t>(i % dim);
    const uint32_t sd = dim / pq_dim;
    const uint32_t sub = d / sd;
    const uint32_t nib = (codes[row * code_size + sub / 2] >> (4 * (sub & 1))) & 15U;
    out[i] = codebooks[(static_cast<uint64_t>(sub) * kPqCentroids + nib) * sd + d % sd];
}

// ProcessQueryImpl (pq_fastscan_quantizer.cpp:299-361), one workgroup per query row.  The float table sits in LDS
// (pq_dim * 16 floats); its smallest and largest entry give lower and diff (TrainUniform, CLASSIC:
// scalar_quantization_trainer.cpp:47-61,72-86); byte = uint8((v - lower) / diff * 255).  Writes tab_bytes bytes per
// row (zero behind the pq_dim * 16 table bytes, zero rows behind the last query) and {diff, lower} into meta.
__global__ void __launch_bounds__(256)
pqfs_query_kernel(const float* q, uint64_t nq, uint32_t dim, uint32_t pq_dim, const float* codebooks, int metric,
                  uint8_t* tab, uint64_t tab_stride, uint32_t tab_bytes, float* meta, uint64_t meta_stride,
                  uint32_t meta_floats) {
    extern __shared__ float lut[];
    __shared__ float red_lo[4], red_hi[4];
    __shared__ float s_norm;
    const uint64_t row = blockIdx.x;
    uint8_t* out = tab + row * tab_stride;
    const uint32_t entries = pq_dim * kPqCentroids;
    if (row >= nq) {
        for (uint32_t e = threadIdx.x; e < tab_bytes; e += blockDim.x) {
            out[e] = 0;
        }
        if (threadIdx.x < meta_floats) {
            meta[row * meta_stride + threadIdx.x] = 0.0F;
        }
        return;
    }
    const float* src = q + row * dim;
    const bool cosine = metric == VSAG_AMD_METRIC_COSINE;
    if (cosine) {
        if (threadIdx.x == 0) {
            float s = 0.0F;
            for (uint32_t d = 0; d < dim; ++d) {
                s = src[d] * src[d] + s;
            }
            const float v = sqrtf(s);
            s_norm = v == 0.0F ? 1.0F : v;
        }
        __syncthreads();
    }
    const float scalar = cosine ? s_norm : 1.0F;
    const uint32_t sd = dim / pq_dim;
    float lo = 3.402823466e+38F, hi = -3.402823466e+38F;
    for (uint32_t e = threadIdx.x; e < entries; e += blockDim.x) {
        const float* c = codebooks + static_cast<uint64_t>(e) * sd;
        const float* qs = src + static_cast<uint64_t>(e / kPqCentroids) * sd;
        float s = 0.0F;
        for (uint32_t d = 0; d < sd; ++d) {
            const float v = cosine ? qs[d] / scalar : qs[d];
            if (metric == VSAG_AMD_METRIC_L2) {
                const float t = v - c[d];
                s = t * t + s;
            } else {
                s = c[d] * v + s;
            }
        }
        lut[e] = s;
        lo = fminf(lo, s);
        hi = fmaxf(hi, s);
    }
    for (int off = 32; off > 0; off >>= 1) {
        lo = fminf(lo, __shfl_xor(lo, off));
        hi = fmaxf(hi, __shfl_xor(hi, off));
    }
    if ((threadIdx.x & 63) == 0) {
        red_lo[threadIdx.x >> 6] = lo;
        red_hi[threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    const float lower = fminf(fminf(red_lo[0], red_lo[1]), fminf(red_lo[2], red_lo[3]));
    const float upper = fmaxf(fmaxf(red_hi[0], red_hi[1]), fmaxf(red_hi[2], red_hi[3]));
    const float diff = upper - lower;
    for (uint32_t e = threadIdx.x; e < tab_bytes; e += blockDim.x) {
        uint32_t byte = 0;
        if (e < entries) {
            const float v = (lut[e] - lower) / diff * 255.0F;
            byte = v == v ? static_cast<uint32_t>(v) & 0xFFU : 0U;  // 0 / 0 (every entry equal): 0
        }
        out[e] = static_cast<uint8_t>(byte);
    }
    if (threadIdx.x == 0) {
        meta[row * meta_stride] = diff;
        meta[row * meta_stride + 1] = lower;
        for (uint32_t m = 2; m < meta_floats; ++m) {
            meta[row * meta_stride + m] = 0.0F;
        }
    }
}

// Package32 / Unpack32 (pq_fastscan_quantizer.cpp:241-297): a block of 32 codes in the order the reference's
// PQFastScanLookUp32 reads them -- subspace i takes 16 bytes, byte j / 2 holds the code of vector MAPPER[j] in its low
// (even j) or high (odd j) nibble; vectors at or beyond `n` read as code 0.  One thread per packaged byte.
__device__ inline uint32_t
pq_mapper(uint32_t j) {
    // {0, 16, 8, 24, 1, 17, 9, 25, ...}: vector = j / 4 + 16 (j % 2) + 8 ((j / 2) % 2)
    return (j >> 2) + 16U * (j & 1U) + 8U * ((j >> 1) & 1U);
}

__global__ void __launch_bounds__(256)
pqfs_package_kernel(const uint8_t* codes, uint64_t n, uint32_t pq_dim, uint32_t code_size, uint8_t* packaged) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint64_t blocks = (n + 31) / 32;
    const uint64_t per_block = static_cast<uint64_t>(code_size) * 32;
    if (i >= blocks * per_block) {
        return;
    }
    const uint64_t blk = i / per_block;
    const uint32_t at = static_cast<uint32_t>(i % per_block);
    const uint32_t sub = at / 16, jb = at % 16;
    uint32_t byte = 0;
    if (sub < pq_dim) {
        for (uint32_t h = 0; h < 2; ++h) {
            const uint64_t v = blk * 32 + pq_mapper(2 * jb + h);
            if (v < n) {
                const uint32_t nib = (codes[v * code_size + sub / 2] >> (4 * (sub & 1))) & 15U;
                byte |= nib << (4 * h);
            }
        }
    }
    packaged[i] = static_cast<uint8_t>(byte);
}

// One thread per plain code byte of the padded blocks.
__global__ void __launch_bounds__(256)
pqfs_unpack_kernel(const uint8_t* packaged, uint64_t n, uint32_t pq_dim, uint32_t code_size, uint8_t* codes) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n * code_size) {
        return;
    }
    const uint64_t v = i / code_size;
    const uint32_t b = static_cast<uint32_t>(i % code_size);
    const uint64_t blk = v / 32;
    const uint32_t lane = static_cast<uint32_t>(v % 32);
    // the j with MAPPER[j] == lane
    const uint32_t j = 4 * (lane & 7U) + (lane >> 4) + 2U * ((lane >> 3) & 1U);
    uint32_t byte = 0;
    for (uint32_t h = 0; h < 2; ++h) {
        const uint32_t sub = 2 * b + h;
        if (sub < pq_dim) {
            const uint32_t pb = packaged[blk * code_size * 32 + sub * 16 + j / 2];
            byte |= ((pb >> (4 * (j & 1U))) & 15U) << (4 * h);
        }
    }
    codes[i] = static_cast<uint8_t>(byte);
}

static int
check_pq(uint32_t dim, uint32_t pq_dim) {
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(pq_dim >= 1 && dim % pq_dim == 0, "pq_dim(%u) does not divide evenly into dim(%u)", pq_dim, dim);
    VA_CHECK_ARG(pq_dim <= kMaxPqDim, "pq_dim must be at most %u, got %u", kMaxPqDim, pq_dim);
    return 0;
}

int
pq_row_norms(const float* x, uint64_t n, uint32_t dim, float* norm, hipStream_t st) {
    hipLaunchKernelGGL(pq_row_norm_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, x, n, dim, norm);
    VA_HIP(hipGetLastError());
    return 0;
}

// The query tables of a pqfs store as the scans read them: per query G * 512 table bytes (16 per subspace, zero behind
// the last subspace) in qtab and {diff, lower} in qmeta.
int
pqfs_prepare_launch(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, uint32_t* qtab,
                    uint32_t qstride, float* qmeta, uint32_t qmeta_stride, hipStream_t st) {
    const size_t lds = static_cast<size_t>(s->pq_dim) * kPqCentroids * sizeof(float);
    hipLaunchKernelGGL(pqfs_query_kernel, dim3(static_cast<uint32_t>(nq_pad)), dim3(256), lds, st, queries, nq, s->dim,
                       s->pq_dim, s->codebooks_dev, s->metric, reinterpret_cast<uint8_t*>(qtab),
                       static_cast<uint64_t>(qstride) * 4, qstride * 4, qmeta, static_cast<uint64_t>(qmeta_stride),
                       qmeta_stride);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_pq_train_workspace_bytes(uint64_t n, uint32_t dim, uint32_t pq_dim) {
    if (pq_dim == 0 || dim % pq_dim != 0 || ensure_init() != 0) {
        return 0;
    }
    const uint64_t count = n < 65536 ? n : 65536;
    const uint32_t sd = dim / pq_dim;
    Carver c(nullptr, 0);
    c.take<float>(count);                  // norms
    c.take<float>(count * sd);             // slice
    c.take<int32_t>(count);                // labels
    const size_t a = vsag_amd_kmeans_init_plus_plus_workspace_bytes(count);
    const size_t b = vsag_amd_kmeans_run_workspace_bytes(count, sd, kPqCentroids);
    c.take<uint8_t>(a > b ? a : b);
    return c.used + 256;
}

// PQFastScanQuantizer::TrainImpl (pq_fastscan_quantizer.cpp:62-94): the first min(n, 65536) rows (normalised for
// cosine), sliced per subspace, 16 centroids by KMeansCluster::Run (k-means++ seeding, 25 Lloyd iterations).  The
// reference seeds from std::random_device; here subspace i draws from mt19937(seed + i): first the row of centroid 0,
// then the 15 k-means++ draws; the Lloyd run re-seeds empty clusters from mt19937(seed + i).  Blocking.
extern "C" int
vsag_amd_pq_train(const float* x_dev, uint64_t n, uint32_t dim, uint32_t pq_dim, int metric, uint64_t seed,
                  float* codebooks_dev, void* workspace_dev, size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_pq(dim, pq_dim));
    VA_CHECK_ARG(x_dev != nullptr && codebooks_dev != nullptr, "null pointer");
    const uint64_t count = n < 65536 ? n : 65536;
    VA_CHECK_ARG(count >= kPqCentroids, "pq training needs at least %u rows, got %llu", kPqCentroids,
                 static_cast<unsigned long long>(n));
    const uint32_t sd = dim / pq_dim;
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver c(workspace_dev, workspace_bytes);
    float* norms = c.take<float>(count);
    float* slice = c.take<float>(count * sd);
    int32_t* labels = c.take<int32_t>(count);
    const size_t wa = vsag_amd_kmeans_init_plus_plus_workspace_bytes(count);
    const size_t wb = vsag_amd_kmeans_run_workspace_bytes(count, sd, kPqCentroids);
    const size_t wk = wa > wb ? wa : wb;
    uint8_t* kws = c.take<uint8_t>(wk);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    const bool cosine = metric == VSAG_AMD_METRIC_COSINE;
    if (cosine) {
        VA_TRY(pq_row_norms(x_dev, count, dim, norms, st));
    }
    for (uint32_t i = 0; i < pq_dim; ++i) {
        hipLaunchKernelGGL(pq_slice_kernel, dim3(static_cast<uint32_t>(div_up(count * sd, 256))), dim3(256), 0, st, x_dev,
                           count, dim, i * sd, sd, cosine ? norms : nullptr, slice);
        VA_HIP(hipGetLastError());
        std::mt19937 gen(static_cast<uint32_t>(seed + i));
        std::uniform_int_distribution<uint64_t> first_dis(0, count - 1);
        const uint64_t first = first_dis(gen);
        std::uniform_real_distribution<double> unit(0.0, 1.0);
        double draws[kPqCentroids - 1];
        for (double& d : draws) {
            d = unit(gen);
            d = d < 1.0 ? d : 0.0;
        }
        float* cb = codebooks_dev + static_cast<uint64_t>(i) * kPqCentroids * sd;
        VA_TRY(vsag_amd_kmeans_init_plus_plus(slice, count, sd, kPqCentroids, first, draws, cb, nullptr, kws, wk, st));
        VA_TRY(vsag_amd_kmeans_run(slice, count, sd, cb, kPqCentroids, 25, seed + i, labels, nullptr, kws, wk, st));
    }
    VA_HIP(hipStreamSynchronize(st));
    return 0;
}

// norm_scratch_dev: n floats, needed under the cosine metric only (may be NULL otherwise).
extern "C" int
vsag_amd_pq_encode(const float* x_dev, uint64_t n, uint32_t dim, uint32_t pq_dim, const float* codebooks_dev, int metric,
                   uint8_t* codes_dev, float* norm_scratch_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_pq(dim, pq_dim));
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(x_dev && codebooks_dev && codes_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t cs = (pq_dim + 1) / 2;
    const bool cosine = metric == VSAG_AMD_METRIC_COSINE;
    if (cosine) {
        VA_CHECK_ARG(norm_scratch_dev != nullptr, "pq encoding under cosine needs n floats of scratch");
        VA_TRY(pq_row_norms(x_dev, n, dim, norm_scratch_dev, st));
    }
    hipLaunchKernelGGL(pq_encode_kernel, dim3(static_cast<uint32_t>(div_up(n * cs, 256))), dim3(256), 0, st, x_dev, n, dim,
                       pq_dim, codebooks_dev, cosine ? norm_scratch_dev : nullptr, codes_dev, cs);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_pq_decode(const uint8_t* codes_dev, uint64_t n, uint32_t dim, uint32_t pq_dim, const float* codebooks_dev,
                   float* out_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_pq(dim, pq_dim));
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev && codebooks_dev && out_dev, "null pointer");
    hipLaunchKernelGGL(pq_decode_kernel, dim3(static_cast<uint32_t>(div_up(n * dim, 256))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), codes_dev, n, dim, pq_dim, codebooks_dev, (pq_dim + 1) / 2,
                       out_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

// Processed queries in the reference's layout: nq x (pq_dim * 16 + 8) bytes -- the byte table, then diff and lower.
extern "C" int
vsag_amd_pqfs_process_query(const float* q_dev, uint64_t nq, uint32_t dim, uint32_t pq_dim, const float* codebooks_dev,
                            int metric, uint8_t* qcodes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_pq(dim, pq_dim));
    if (nq == 0) {
        return 0;
    }
    VA_CHECK_ARG(q_dev && codebooks_dev && qcodes_dev, "null pointer");
    VA_CHECK_ARG(nq <= 0x7FFFFFFFull, "too many queries");
    const uint64_t stride = static_cast<uint64_t>(pq_dim) * kPqCentroids + 8;
    const size_t lds = static_cast<size_t>(pq_dim) * kPqCentroids * sizeof(float);
    hipLaunchKernelGGL(pqfs_query_kernel, dim3(static_cast<uint32_t>(nq)), dim3(256), lds, static_cast<hipStream_t>(stream),
                       q_dev, nq, dim, pq_dim, codebooks_dev, metric, qcodes_dev, stride, pq_dim * kPqCentroids,
                       reinterpret_cast<float*>(qcodes_dev + static_cast<uint64_t>(pq_dim) * kPqCentroids), stride / 4, 2U);
    VA_HIP(hipGetLastError());
    return 0;
}

// n codes -> ceil(n / 32) packaged blocks of 32 * code_size bytes, and back.
extern "C" int
vsag_amd_pqfs_package(const uint8_t* codes_dev, uint64_t n, uint32_t pq_dim, uint8_t* packaged_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(pq_dim >= 1 && pq_dim <= kMaxPqDim, "pq_dim must be in [1, %u], got %u", kMaxPqDim, pq_dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev && packaged_dev, "null pointer");
    const uint32_t cs = (pq_dim + 1) / 2;
    const uint64_t bytes = div_up(n, 32) * 32 * cs;
    hipLaunchKernelGGL(pqfs_package_kernel, dim3(static_cast<uint32_t>(div_up(bytes, 256))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), codes_dev, n, pq_dim, cs, packaged_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_pqfs_unpack(const uint8_t* packaged_dev, uint64_t n, uint32_t pq_dim, uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(pq_dim >= 1 && pq_dim <= kMaxPqDim, "pq_dim must be in [1, %u], got %u", kMaxPqDim, pq_dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev && packaged_dev, "null pointer");
    const uint32_t cs = (pq_dim + 1) / 2;
    hipLaunchKernelGGL(pqfs_unpack_kernel, dim3(static_cast<uint32_t>(div_up(n * cs, 256))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), packaged_dev, n, pq_dim, cs, codes_dev);
    VA_HIP(hipGetLastError());
    return 0;
}
