// Quantizer training and encoding on the device: scalar-quantization bounds, sq8/sq4 codes, uniform
// codes, RaBitQ 1-bit codes and processed queries.  These are build-time and per-batch steps, not the
// scan; they are written so that their results equal the reference's scalar arithmetic bit for bit where
// that arithmetic is order-dependent (running fp32 sums are kept in element order, products and sums are
// not fused: this translation unit is compiled with -ffp-contract=off).
#include <cfloat>

#include "common.h"
#include "topk.h"

namespace vsag_amd {

// ------------------------------------------------------------------ helpers
// generic::Normalize (src/simd/generic.cpp:874-878, kernels/scalar_op.h:32-60): ||x|| as a running sum in
// element order; a zero norm divides by one.
__global__ void
row_norm_kernel(const float* x, uint64_t n, uint32_t dim, float* norms) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const float* r = x + i * dim;
    float s = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        s = r[d] * r[d] + s;
    }
    float norm = sqrtf(s);
    norms[i] = norm == 0.0F ? 1.0F : norm;
}

// ClampScalarQuantizationDelta (scalar_quantization_utils.h:19-30).
__device__ inline float
clamp_delta(float delta) {
    if (!(delta >= 0.0F)) {
        return 0.0F;
    }
    if (delta > 0.999F) {
        return 1.0F;
    }
    return delta;
}

// ------------------------------------------------------------------ sq8 / sq4 encode
// ScalarQuantizer::EncodeOneImpl (scalar_quantizer.cpp:85-112).  One thread per code byte.
__global__ void __launch_bounds__(256)
sq_encode_kernel(const float* x, uint64_t n, uint32_t dim, int bits, const float* lb, const float* diff,
                 const float* norms, uint32_t code_size, uint8_t* codes) {
    uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint64_t i = gid / code_size;
    uint32_t b = static_cast<uint32_t>(gid % code_size);
    if (i >= n) {
        return;
    }
    const float* r = x + i * dim;
    float inv = norms ? norms[i] : 1.0F;
    float levels = static_cast<float>((1 << bits) - 1);
    uint32_t per_byte = 8 / bits;
    uint32_t byte = 0;
    for (uint32_t e = 0; e < per_byte; ++e) {
        uint32_t d = b * per_byte + e;
        if (d >= dim) {
            break;
        }
        float v = norms ? r[d] / inv : r[d];
        float delta;
        if (diff[d] < FLT_EPSILON) {
            delta = 1.0F;
        } else {
            delta = 1.0F * (v - lb[d]) / diff[d];
        }
        delta = clamp_delta(delta);
        uint32_t scaled = static_cast<uint8_t>(levels * delta);
        byte |= scaled << (e * bits);
    }
    codes[i * code_size + b] = static_cast<uint8_t>(byte);
}

// ------------------------------------------------------------------ uniform encode
// SQ4UniformQuantizer::EncodeOneImpl / SQ8UniformQuantizer::EncodeOneImpl.  One wave per row; the integer
// norm is order-free, the two fp32 sums are accumulated by lane 0 in element order.
__global__ void __launch_bounds__(256)
squ_encode_kernel(const float* x, uint64_t n, uint32_t dim, int bits, int metric, const float* bounds,
                  const float* norms, uint32_t code_size, uint32_t payload, uint32_t off_norm, uint32_t off_sum,
                  uint32_t off_codes_sum, uint8_t* codes) {
    uint64_t row = static_cast<uint64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    uint32_t lane = threadIdx.x & 63;
    if (row >= n) {
        return;
    }
    const float* r = x + row * dim;
    uint8_t* c = codes + row * code_size;
    float lb = bounds[0], diff = bounds[1];
    float inv_diff = diff == 0.0F ? 0.0F : 1.0F / diff;
    float levels = bits == 4 ? 15.0F : 255.0F;
    float nrm = norms ? norms[row] : 1.0F;
    uint32_t per_byte = 8 / bits;
    uint32_t norm_part = 0;
    for (uint32_t b = lane; b < code_size; b += kWave) {
        uint32_t byte = 0;
        if (b < payload) {
            for (uint32_t e = 0; e < per_byte; ++e) {
                uint32_t d = b * per_byte + e;
                if (d >= dim) {
                    break;
                }
                float v = norms ? r[d] / nrm : r[d];
                float delta = clamp_delta((v - lb) * inv_diff);
                uint32_t scaled = static_cast<uint8_t>(levels * delta);
                byte |= scaled << (e * bits);
                norm_part += scaled * scaled;
            }
        }
        c[b] = static_cast<uint8_t>(byte);
    }
    for (int off = 32; off > 0; off >>= 1) {
        norm_part += __shfl_down(norm_part, off);
    }
    // All lanes have written their bytes; lane 0 overwrites the trailing fields.
    wave_lds_fence();
    if (lane == 0) {
        if (metric == VSAG_AMD_METRIC_L2) {
            uint64_t v = norm_part;
            for (int b = 0; b < 8; ++b) {
                c[off_norm + b] = static_cast<uint8_t>(v >> (8 * b));
            }
        } else {
            float sum = 0.0F, codes_sum = 0.0F;
            for (uint32_t d = 0; d < dim; ++d) {
                float v = norms ? r[d] / nrm : r[d];
                float delta = clamp_delta((v - lb) * inv_diff);
                uint32_t scaled = static_cast<uint8_t>(levels * delta);
                sum += v;
                codes_sum += static_cast<float>(scaled);
            }
            uint32_t u = __float_as_uint(sum);
            for (int b = 0; b < 4; ++b) {
                c[off_sum + b] = static_cast<uint8_t>(u >> (8 * b));
            }
            if (bits == 4) {
                u = __float_as_uint(codes_sum);
                for (int b = 0; b < 4; ++b) {
                    c[off_codes_sum + b] = static_cast<uint8_t>(u >> (8 * b));
                }
            }
        }
    }
}

// ------------------------------------------------------------------ C = A * B^T, k in element order
// C[i][j] = sum_k A[i][k] * B[j][k], one unfused multiply and add per k in increasing k, so every output
// equals a scalar running-sum dot product (the RowMajor sgemv of random_orthogonal_transformer.cpp:58-77
// restated in element order).  64 x 64 output tile per workgroup, 4 x 4 outputs per thread.
__global__ void __launch_bounds__(256)
gemm_nt_seq_kernel(const float* A, const float* B, float* C, uint64_t M, uint32_t N, uint32_t K) {
    __shared__ float As[16][65];
    __shared__ float Bs[16][65];
    const uint32_t tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.y) * 64;
    const uint32_t col0 = blockIdx.x * 64;
    float acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < K; k0 += 16) {
        for (uint32_t idx = threadIdx.x; idx < 64 * 16; idx += 256) {
            uint32_t r = idx >> 4, kk = idx & 15;
            uint64_t ar = row0 + r;
            uint32_t br = col0 + r;
            As[kk][r] = (ar < M && k0 + kk < K) ? A[ar * K + k0 + kk] : 0.0F;
            Bs[kk][r] = (br < N && k0 + kk < K) ? B[static_cast<uint64_t>(br) * K + k0 + kk] : 0.0F;
        }
        __syncthreads();
        uint32_t kmax = K - k0 < 16 ? K - k0 : 16;
        for (uint32_t kk = 0; kk < kmax; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = As[kk][ty * 4 + i];
                b[i] = Bs[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = a[i] * b[j] + acc[i][j];
                }
            }
        }
        __syncthreads();
    }
    for (int i = 0; i < 4; ++i) {
        uint64_t r = row0 + ty * 4 + i;
        if (r >= M) {
            continue;
        }
        for (int j = 0; j < 4; ++j) {
            uint32_t cidx = col0 + tx * 4 + j;
            if (cidx < N) {
                C[r * N + cidx] = acc[i][j];
            }
        }
    }
}

static int
gemm_nt_seq(const float* A, const float* B, float* C, uint64_t M, uint32_t N, uint32_t K, hipStream_t st) {
    dim3 grid((N + 63) / 64, static_cast<uint32_t>(div_up(M, 64)));
    hipLaunchKernelGGL(gemm_nt_seq_kernel, grid, dim3(256), 0, st, A, B, C, M, N, K);
    VA_HIP(hipGetLastError());
    return 0;
}

// ------------------------------------------------------------------ RaBitQ
struct RabitqLayout {
    uint32_t dim, code_bytes;
    uint32_t base_bits, offset_norm_code;  // bits per dimension of the base code; |code - centre| where base_bits != 1
    uint32_t offset_norm, offset_error, offset_sum, offset_raw_norm, code_size;
    int has_sum, has_raw_norm;
    uint32_t aligned_dim, plane_bytes;
    uint32_t q_offset_lb, q_offset_delta, q_offset_sum, q_offset_norm, q_offset_raw_norm, query_code_size;
};

// rabitq_quantizer.cpp:102-176 (standard version, no PCA / MRQ / split storage).  `query_bits` is the bits word of the
// C interface: 4 or 32 for the query, plus 256 * base bits for multi-bit base codes (VSAG_AMD_RABITQ_BITS).
__host__ __device__ inline RabitqLayout
rabitq_layout(uint32_t dim, int metric, int query_bits) {
    RabitqLayout l{};
    l.dim = dim;
    l.base_bits = (query_bits >> 8) == 0 ? 1U : static_cast<uint32_t>(query_bits >> 8);
    query_bits &= 255;
    l.code_bytes = (dim + 7) / 8 * l.base_bits;
    uint32_t cs = (l.code_bytes + 3) / 4 * 4;
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
    l.has_raw_norm = metric != VSAG_AMD_METRIC_L2;
    if (l.has_raw_norm) {
        l.offset_raw_norm = cs;
        cs += 4;
    }
    l.code_size = cs;
    uint32_t qs;
    if (query_bits == 4) {
        l.aligned_dim = (dim + 511) / 512 * 512;
        l.plane_bytes = l.aligned_dim / 8;
        qs = l.plane_bytes * 4;
        l.q_offset_lb = qs;
        qs += 4;
        l.q_offset_delta = qs;
        qs += 4;
        l.q_offset_sum = qs;
        qs += 4;
    } else {
        qs = 4 * dim;
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

uint64_t
rabitq_code_size(uint32_t dim, int metric, int query_bits) {
    return rabitq_layout(dim, metric, query_bits).code_size;
}
uint64_t
rabitq_query_code_size(uint32_t dim, int metric, int query_bits) {
    return rabitq_layout(dim, metric, query_bits).query_code_size;
}

__device__ inline float
load_f32(const uint8_t* p) {
    uint32_t u = 0;
    for (int b = 0; b < 4; ++b) {
        u |= static_cast<uint32_t>(p[b]) << (8 * b);
    }
    return __uint_as_float(u);
}

__device__ inline void
store_f32(uint8_t* p, float v) {
    uint32_t u = __float_as_uint(v);
    for (int b = 0; b < 4; ++b) {
        p[b] = static_cast<uint8_t>(u >> (8 * b));
    }
}

// Column means as running fp32 sums over the rows in order (rabitq_quantizer.cpp:224-241).  A workgroup owns 32
// columns: all 1024 threads stage the next 256 rows of those columns in LDS while the first 32 threads add the
// current 256 rows, one column each, in row order -- the additions stay sequential, the loads do not.
constexpr uint32_t kMeanCols = 32;
constexpr uint32_t kMeanRows = 256;

__global__ void __launch_bounds__(1024)
column_mean_seq_kernel(const float* x, uint64_t n, uint32_t dim, float* mean) {
    __shared__ float stage[2][kMeanRows][kMeanCols];
    const uint32_t col = threadIdx.x & (kMeanCols - 1);
    const uint32_t slot = threadIdx.x / kMeanCols;  // 0..31
    const uint32_t d = blockIdx.x * kMeanCols + col;
    const bool live = d < dim;
    float regs[kMeanRows / 32];
    auto fetch = [&](uint64_t row0) {
#pragma unroll
        for (uint32_t u = 0; u < kMeanRows / 32; ++u) {
            uint64_t r = row0 + u * 32 + slot;
            regs[u] = live && r < n ? x[r * dim + d] : 0.0F;
        }
    };
    auto park = [&](uint32_t b) {
#pragma unroll
        for (uint32_t u = 0; u < kMeanRows / 32; ++u) {
            stage[b][u * 32 + slot][col] = regs[u];
        }
    };
    fetch(0);
    park(0);
    __syncthreads();
    float s = 0.0F;
    uint32_t b = 0;
    for (uint64_t row0 = 0; row0 < n; row0 += kMeanRows, b ^= 1) {
        const bool more = row0 + kMeanRows < n;
        if (more) {
            fetch(row0 + kMeanRows);
        }
        if (slot == 0) {
            uint32_t m = n - row0 < kMeanRows ? static_cast<uint32_t>(n - row0) : kMeanRows;
            for (uint32_t r = 0; r < m; ++r) {
                s += stage[b][r][col];
            }
        }
        if (more) {
            park(b ^ 1);
        }
        __syncthreads();
    }
    if (slot == 0 && live) {
        mean[d] = s / static_cast<float>(n);
    }
}

// Second half of RaBitQuantizer::EncodeOneInternal (rabitq_quantizer.cpp:749-856) for rows already rotated:
// raw norm of the input row, NormalizeWithCentroid (kernels/normalize.h:35-83), sign bits, error =
// RaBitQFloatBinaryIP(normed, bits) (generic.cpp:447-471), bit count.  One thread per row, element order.
__global__ void __launch_bounds__(64)
rabitq_finish_encode_kernel(const float* raw, const float* rotated, uint64_t n, uint32_t dim, const float* centroid,
                            int metric, int query_bits, uint8_t* codes) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    const float* y = rotated + i * dim;
    uint8_t* c = codes + i * l.code_size;
    float raw_norm = 0.0F;
    if (l.has_raw_norm) {
        const float* x = raw + i * dim;
        for (uint32_t d = 0; d < dim; ++d) {
            raw_norm += x[d] * x[d];
        }
    }
    raw_norm = sqrtf(raw_norm);
    float norm_sq = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        float t = y[d] - centroid[d];
        norm_sq = t * t + norm_sq;
    }
    float norm = norm_sq < 1e-5F ? 1.0F : sqrtf(norm_sq);
    float inv_sqrt_d = 1.0F / sqrtf(static_cast<float>(dim));
    float pos, neg;
    if (inv_sqrt_d > 1e-3F) {
        pos = inv_sqrt_d;
        neg = -inv_sqrt_d;
    } else {
        pos = 1.0F;
        neg = 0.0F;
    }
    float error = 0.0F;
    uint32_t binary_sum = 0;
    for (uint32_t b = 0; b < l.offset_norm; ++b) {
        uint32_t byte = 0;
        for (uint32_t e = 0; e < 8; ++e) {
            uint32_t d = b * 8 + e;
            if (d >= dim) {
                break;
            }
            float nd = (y[d] - centroid[d]) / norm;
            bool bit = nd >= 0.0F;
            if (bit) {
                byte |= 1U << e;
                ++binary_sum;
            }
            error += (bit ? pos : neg) * nd;
        }
        c[b] = static_cast<uint8_t>(byte);
    }
    store_f32(c + l.offset_norm, norm);
    store_f32(c + l.offset_error, error);
    if (l.has_sum) {
        store_f32(c + l.offset_sum, static_cast<float>(binary_sum));
    }
    if (l.has_raw_norm) {
        store_f32(c + l.offset_raw_norm, raw_norm);
    }
}

// ---- multi-bit base codes (rabitq_bits_per_dim_base 2..8) ----
// Norm of (rotated row - centroid) as NormalizeWithCentroid takes it (kernels/normalize.h:35-83).
__device__ inline float
rabitq_row_norm(const float* y, const float* centroid, uint32_t dim) {
    float norm_sq = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        float t = y[d] - centroid[d];
        norm_sq = t * t + norm_sq;
    }
    return norm_sq < 1e-5F ? 1.0F : sqrtf(norm_sq);
}

// RaBitQuantizer::FastEncodeRaBitQ (rabitq_quantizer.cpp:609-704): a floor grid over [-max|o|, max|o|], then `rounds`
// sweeps of one-level moves per coordinate that raise <o, y>^2 / |y|^2 (y = code - centre).  The sweep is sequential
// per row (every move changes the sums the next coordinate is judged by), so one thread owns a row; all sums are
// doubles in the reference's order.  scalar: n x dim code values; norm_code: n floats.
__global__ void __launch_bounds__(64)
rabitq_fast_encode_kernel(const float* rotated, uint64_t n, uint32_t dim, const float* centroid, uint32_t bits,
                          uint32_t rounds, uint8_t* scalar, float* norm_code) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const float* y = rotated + i * dim;
    uint8_t* code = scalar + i * dim;
    const float norm = rabitq_row_norm(y, centroid, dim);
    const uint32_t code_max = (1U << bits) - 1U;
    const double center = 0.5 * static_cast<double>(code_max);
    double max_abs = 0.0;
    for (uint32_t d = 0; d < dim; ++d) {
        const float o = (y[d] - centroid[d]) / norm;
        max_abs = fmax(max_abs, fabs(static_cast<double>(o)));
    }
    if (max_abs <= 0.0) {
        for (uint32_t d = 0; d < dim; ++d) {
            code[d] = static_cast<uint8_t>(code_max / 2U);
        }
        norm_code[i] = 1.0F;
        return;
    }
    const double delta = 2.0 * max_abs / static_cast<double>(code_max + 1U);
    const double inv_delta = 1.0 / delta;
    double ip = 0.0, norm_sqr = 0.0;
    for (uint32_t d = 0; d < dim; ++d) {
        const float o = (y[d] - centroid[d]) / norm;
        const double scaled = (static_cast<double>(o) + max_abs) * inv_delta;
        long long q = static_cast<long long>(floor(scaled));
        q = q < 0 ? 0 : (q > static_cast<long long>(code_max) ? static_cast<long long>(code_max) : q);
        code[d] = static_cast<uint8_t>(q);
        const double centered = static_cast<double>(q) - center;
        ip += static_cast<double>(o) * centered;
        norm_sqr += centered * centered;
    }
    for (uint32_t round = 0; round < rounds; ++round) {
        bool adjusted = false;
        for (uint32_t d = 0; d < dim; ++d) {
            const double o = static_cast<double>((y[d] - centroid[d]) / norm);
            const int cur = code[d];
            const double cur_value = static_cast<double>(cur) - center;
            int best_code = cur;
            double best_ip = ip, best_norm = norm_sqr;
            double best_score = norm_sqr > 0.0 ? ip * ip / norm_sqr : 0.0;
#pragma unroll
            for (int dir = -1; dir <= 1; dir += 2) {
                const int cand = cur + dir;
                if (cand < 0 || cand > static_cast<int>(code_max)) {
                    continue;
                }
                const double cand_ip = ip + static_cast<double>(dir) * o;
                if (cand_ip < 0.0) {
                    continue;
                }
                const double cand_norm = norm_sqr + 2.0 * cur_value * static_cast<double>(dir) + 1.0;
                const double cand_score = cand_norm > 0.0 ? cand_ip * cand_ip / cand_norm : 0.0;
                const double tolerance = 1e-8 * fmax(1.0, fabs(best_score));
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
    for (uint32_t d = 0; d < dim; ++d) {
        const double centered = static_cast<double>(code[d]) - center;
        norm_sqr += centered * centered;
    }
    float yn = static_cast<float>(sqrt(norm_sqr));
    if (!isfinite(yn) || yn <= 0.0F) {
        yn = 1.0F;
    }
    norm_code[i] = yn;
}

// RaBitQuantizer::EncodeExtendRaBitQ (rabitq_quantizer.cpp:455-607): the scale t walks upwards, one grid step of one
// coordinate per event, events in (t, coordinate) order -- the reference's priority queue always holds at most one
// pending event per coordinate, so "pop" is the minimum over the coordinates' next event times.  One wave per row:
// the lanes share that minimum search, every lane repeats the running sums (doubles, the reference's order).
// LDS per row: dim doubles (next event), dim ints (grid position), dim floats (o).
__global__ void __launch_bounds__(64)
rabitq_extend_encode_kernel(const float* rotated, uint64_t n, uint32_t dim, const float* centroid, uint32_t bits,
                            uint8_t* scalar, float* norm_code) {
    extern __shared__ double ee_lds[];
    double* next_t = ee_lds;
    int* y2_cur = reinterpret_cast<int*>(next_t + dim);
    float* o = reinterpret_cast<float*>(y2_cur + dim);
    const uint64_t i = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const float* y = rotated + i * dim;
    uint8_t* code = scalar + i * dim;
    float norm = 0.0F;
    if (lane == 0) {
        norm = rabitq_row_norm(y, centroid, dim);
    }
    norm = __shfl(norm, 0);
    const int y2_max = static_cast<int>((1U << bits) - 1U);
    const double c = 0.5 * static_cast<double>(y2_max);
    const double inf = __builtin_huge_val();
    double max_o = 0.0;
    for (uint32_t d = lane; d < dim; d += kWave) {
        const float v = (y[d] - centroid[d]) / norm;
        o[d] = v;
        max_o = fmax(max_o, fabs(static_cast<double>(v)));
    }
    for (int off = 32; off > 0; off >>= 1) {
        max_o = fmax(max_o, __shfl_xor(max_o, off));
    }
    if (max_o <= 0.0) {
        for (uint32_t d = lane; d < dim; d += kWave) {
            code[d] = static_cast<uint8_t>(y2_max / 2);
        }
        if (lane == 0) {
            norm_code[i] = 1.0F;
        }
        return;
    }
    const double t_end = (static_cast<double>(y2_max) + 2.0) / (2.0 * max_o);
    // Next event time of a coordinate at grid position `pos` (compute_next_t_for_dim, :513-531).
    auto next_event = [&](double oi, int pos) {
        if (fabs(oi) < 1e-3) {
            return inf;
        }
        const int sign = (oi > 0.0) ? +1 : -1;
        const int y2_next = pos + sign * 2;
        if (y2_next < -y2_max || y2_next > +y2_max) {
            return inf;
        }
        double t = static_cast<double>(pos + sign) / (2.0 * oi);
        if (t < 0.0) {
            t = 0.0;
        }
        return t;
    };
    for (uint32_t d = lane; d < dim; d += kWave) {
        const double oi = static_cast<double>(o[d]);
        double t0 = inf;
        if (oi != 0.0) {
            t0 = next_event(oi, 0);
            if (!(t0 <= t_end)) {
                t0 = inf;
            }
        }
        next_t[d] = t0;
        y2_cur[d] = 0;
    }
    wave_lds_fence();
    double ip_y2_o = 0.0, norm_y2 = 0.0;
    double best_ip = 1e-12, best_t = 0.0;
    // Every pass retires one event; a coordinate has at most 2^(bits - 1) of them, so the walk ends.
    const uint64_t max_events = static_cast<uint64_t>(dim) << bits;
    for (uint64_t ev = 0; ev < max_events; ++ev) {
        double bt = inf;
        uint32_t bi = 0xFFFFFFFFU;
        for (uint32_t d = lane; d < dim; d += kWave) {
            const double t = next_t[d];
            if (t < bt) {
                bt = t;
                bi = d;
            }
        }
        for (int off = 32; off > 0; off >>= 1) {
            const double ot = __shfl_xor(bt, off);
            const uint32_t oi = __shfl_xor(bi, off);
            if (ot < bt || (ot == bt && oi < bi)) {
                bt = ot;
                bi = oi;
            }
        }
        if (bi == 0xFFFFFFFFU || !(bt < t_end)) {
            break;
        }
        const double cur_t = bt;
        const uint32_t k = bi;
        const double ok = static_cast<double>(o[k]);
        const int sign = (o[k] > 0.0F) ? +1 : -1;
        const int y2_old = y2_cur[k];
        const int y2_new = y2_old + sign * 2;
        wave_lds_fence();
        if (y2_new < -y2_max || y2_new > +y2_max) {
            if (lane == 0) {
                next_t[k] = inf;
            }
            wave_lds_fence();
            continue;
        }
        ip_y2_o += (static_cast<double>(y2_new) - static_cast<double>(y2_old)) * ok;
        norm_y2 += static_cast<double>(y2_new) * static_cast<double>(y2_new) -
                   static_cast<double>(y2_old) * static_cast<double>(y2_old);
        const double cur_ip = (norm_y2 > 0.0) ? (ip_y2_o / sqrt(norm_y2)) : 0.0;
        if (cur_ip > best_ip) {
            best_ip = cur_ip;
            best_t = cur_t;
        }
        double t_next = next_event(ok, y2_new);
        if (t_next <= cur_t) {
            t_next = __longlong_as_double(__double_as_longlong(cur_t) + 1);  // nextafter(cur_t, +inf), cur_t >= 0
        }
        if (lane == 0) {
            y2_cur[k] = y2_new;
            next_t[k] = (t_next < t_end) ? t_next : inf;  // a finite time below the end, else no further event
        }
        wave_lds_fence();
    }
    double sum_y2 = 0.0;  // a sum of k + 0.25 terms: exact in any order
    for (uint32_t d = lane; d < dim; d += kWave) {
        const double val = 2.0 * best_t * static_cast<double>(o[d]);
        const double shifted = val + ((val >= 0) ? 1e-12 : -1e-12);
        long long r = llround(shifted);
        int ri = r < -y2_max ? -y2_max : (r > y2_max ? y2_max : static_cast<int>(r));
        if ((ri & 1) != (y2_max & 1)) {
            const int step = (shifted >= 0.0) ? +1 : -1;
            int cand = ri + step;
            if (cand < -y2_max || cand > y2_max) {
                cand = ri - step;
            }
            ri = cand < -y2_max ? -y2_max : (cand > y2_max ? y2_max : cand);
        }
        int u = (ri + y2_max) / 2;
        u = u < 0 ? 0 : (u > y2_max ? y2_max : u);
        code[d] = static_cast<uint8_t>(u);
        const double yy = static_cast<double>(u) - c;
        sum_y2 += yy * yy;
    }
    for (int off = 32; off > 0; off >>= 1) {
        sum_y2 += __shfl_xor(sum_y2, off);
    }
    if (lane == 0) {
        float yn = static_cast<float>(sqrt(sum_y2));
        if (!isfinite(yn) || yn <= 0.0F) {
            yn = 1.0F;
        }
        norm_code[i] = yn;
    }
}

// Rest of the multi-bit branch of RaBitQuantizer::EncodeOneInternal (rabitq_quantizer.cpp:789-809, 852-855): bit planes
// (PackIntoPlanes, :431-453: plane b holds bit b of every dimension), |code - centre|, the norms, and error =
// ip_obar_q(<o, code>, sum o, |code - centre|) with both sums as running floats in element order.  One thread per row.
__global__ void __launch_bounds__(64)
rabitq_multibit_finish_kernel(const float* raw, const float* rotated, uint64_t n, uint32_t dim, const float* centroid,
                              int metric, int bits_word, const uint8_t* scalar, const float* norm_code,
                              uint8_t* codes) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const RabitqLayout l = rabitq_layout(dim, metric, bits_word);
    const float* y = rotated + i * dim;
    const uint8_t* sc = scalar + i * dim;
    uint8_t* c = codes + i * l.code_size;
    float raw_norm = 0.0F;
    if (l.has_raw_norm) {
        const float* x = raw + i * dim;
        for (uint32_t d = 0; d < dim; ++d) {
            raw_norm += x[d] * x[d];
        }
    }
    raw_norm = sqrtf(raw_norm);
    const float norm = rabitq_row_norm(y, centroid, dim);
    const uint32_t plane_bytes = (dim + 7) / 8;
    float query_sum = 0.0F, scalar_ip = 0.0F;
    for (uint32_t b = 0; b < plane_bytes; ++b) {
        uint32_t plane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t d = b * 8 + e;
            if (d >= dim) {
                break;
            }
            const float nd = (y[d] - centroid[d]) / norm;
            const uint32_t v = sc[d];
            query_sum += nd;
            scalar_ip += static_cast<float>(v) * nd;
#pragma unroll
            for (uint32_t p = 0; p < 8; ++p) {
                plane[p] |= ((v >> p) & 1U) << e;
            }
        }
#pragma unroll
        for (uint32_t p = 0; p < 8; ++p) {
            if (p < l.base_bits) {
                c[p * plane_bytes + b] = static_cast<uint8_t>(plane[p]);
            }
        }
    }
    for (uint32_t b = l.code_bytes; b < l.offset_norm_code; ++b) {
        c[b] = 0;
    }
    const float yn = norm_code[i];
    // ip_obar_q (rabitq_quantizer.cpp:256-267)
    float error = 0.0F;
    if (yn > 0.0F) {
        error = scalar_ip - 0.5F * static_cast<float>((1U << l.base_bits) - 1U) * query_sum;
        error /= yn;
    }
    store_f32(c + l.offset_norm_code, yn);
    store_f32(c + l.offset_norm, norm);
    store_f32(c + l.offset_error, error);
    if (l.has_raw_norm) {
        store_f32(c + l.offset_raw_norm, raw_norm);
    }
}

// Second half of RaBitQuantizer::ProcessQueryImpl (rabitq_quantizer.cpp:2130-2217) with EncodeSQ and
// ReOrderSQ (:2049-2088) for queries already rotated.  One thread per query.
__global__ void __launch_bounds__(64)
rabitq_finish_query_kernel(const float* raw, const float* rotated, uint64_t nq, uint32_t dim, const float* centroid,
                           int metric, int query_bits, uint8_t* qcodes) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= nq) {
        return;
    }
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    const float* y = rotated + i * dim;
    uint8_t* qc = qcodes + i * l.query_code_size;
    float raw_norm = 0.0F;
    if (l.has_raw_norm) {
        const float* x = raw + i * dim;
        for (uint32_t d = 0; d < dim; ++d) {
            raw_norm += x[d] * x[d];
        }
    }
    raw_norm = sqrtf(raw_norm);
    float norm_sq = 0.0F;
    for (uint32_t d = 0; d < dim; ++d) {
        float t = y[d] - centroid[d];
        norm_sq = t * t + norm_sq;
    }
    float norm = norm_sq < 1e-5F ? 1.0F : sqrtf(norm_sq);
    if (l.base_bits != 1) {
        float sum = 0.0F;
        for (uint32_t d = 0; d < dim; ++d) {
            sum += (y[d] - centroid[d]) / norm;
        }
        store_f32(qc + l.q_offset_sum, sum);
    }
    if ((query_bits & 255) == 4) {
        float lb = FLT_MAX, ub = -FLT_MAX;
        for (uint32_t d = 0; d < dim; ++d) {
            float v = (y[d] - centroid[d]) / norm;
            if (v < lb) {
                lb = v;
            }
            if (v > ub) {
                ub = v;
            }
        }
        float delta = (ub - lb) / 15;
        float inv_delta = fabsf(delta) < 1e-5F ? 0.0F : 1.0F / delta;
        float qsum = 0.0F;
        for (uint32_t b = 0; b < l.plane_bytes; ++b) {
            uint32_t plane[4] = {0, 0, 0, 0};
            for (uint32_t e = 0; e < 8; ++e) {
                uint32_t d = b * 8 + e;
                if (d >= dim) {
                    break;
                }
                float v = (y[d] - centroid[d]) / norm;
                float val = roundf((v - lb) * inv_delta);
                uint32_t q = static_cast<uint8_t>(val);
                qsum += static_cast<float>(val);
                for (uint32_t p = 0; p < 4; ++p) {
                    plane[p] |= ((q >> p) & 1U) << e;
                }
            }
            for (uint32_t p = 0; p < 4; ++p) {
                qc[p * l.plane_bytes + b] = static_cast<uint8_t>(plane[p]);
            }
        }
        store_f32(qc + l.q_offset_lb, lb);
        store_f32(qc + l.q_offset_delta, delta);
        store_f32(qc + l.q_offset_sum, qsum);
    } else {
        for (uint32_t d = 0; d < dim; ++d) {
            store_f32(qc + 4 * d, (y[d] - centroid[d]) / norm);
        }
    }
    store_f32(qc + l.q_offset_norm, norm);
    if (l.has_raw_norm) {
        store_f32(qc + l.q_offset_raw_norm, raw_norm);
    }
}

// The same, one wave per query: the loads are coalesced and everything but the two sums whose order matters (the
// squared norms, added dimension by dimension like the reference does) is spread over the lanes.  The sum of the
// quantised values is a sum of small integers, exact in any order.  LDS: dim floats, twice that with a raw norm.
__global__ void __launch_bounds__(64)
rabitq_finish_query_wave_kernel(const float* raw, const float* rotated, uint64_t nq, uint32_t dim, const float* centroid,
                                int metric, int query_bits, uint8_t* qcodes) {
    extern __shared__ float fq_lds[];
    const uint64_t i = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    const float* y = rotated + i * dim;
    uint8_t* qc = qcodes + i * l.query_code_size;
    float* t = fq_lds;        // y - centroid
    float* xx = fq_lds + dim;  // squares of the raw query
    for (uint32_t d = lane; d < dim; d += kWave) {
        t[d] = y[d] - centroid[d];
        if (l.has_raw_norm) {
            const float x = raw[i * dim + d];
            xx[d] = x * x;
        }
    }
    wave_lds_fence();
    float raw_norm = 0.0F, norm_sq = 0.0F;
    if (lane == 0) {
        for (uint32_t d = 0; d < dim; ++d) {
            const float v = t[d];
            norm_sq = v * v + norm_sq;
            if (l.has_raw_norm) {
                raw_norm += xx[d];
            }
        }
    }
    raw_norm = sqrtf(__shfl(raw_norm, 0));
    norm_sq = __shfl(norm_sq, 0);
    const float norm = norm_sq < 1e-5F ? 1.0F : sqrtf(norm_sq);
    if (l.base_bits != 1 && lane == 0) {
        float sum = 0.0F;  // in element order, like the reference (rabitq_quantizer.cpp:2199-2205)
        for (uint32_t d = 0; d < dim; ++d) {
            sum += t[d] / norm;
        }
        store_f32(qc + l.q_offset_sum, sum);
    }
    if ((query_bits & 255) == 4) {
        float lb = FLT_MAX, ub = -FLT_MAX;
        for (uint32_t d = lane; d < dim; d += kWave) {
            const float v = t[d] / norm;
            if (v < lb) {
                lb = v;
            }
            if (v > ub) {
                ub = v;
            }
        }
        for (int off = 32; off > 0; off >>= 1) {
            const float ol = __shfl_xor(lb, off), ou = __shfl_xor(ub, off);
            if (ol < lb) {
                lb = ol;
            }
            if (ou > ub) {
                ub = ou;
            }
        }
        const float delta = (ub - lb) / 15;
        const float inv_delta = fabsf(delta) < 1e-5F ? 0.0F : 1.0F / delta;
        float qsum = 0.0F;
        for (uint32_t b = lane; b < l.plane_bytes; b += kWave) {
            uint32_t plane[4] = {0, 0, 0, 0};
            for (uint32_t e = 0; e < 8; ++e) {
                const uint32_t d = b * 8 + e;
                if (d >= dim) {
                    break;
                }
                const float v = t[d] / norm;
                const float val = roundf((v - lb) * inv_delta);
                const uint32_t q = static_cast<uint8_t>(val);
                qsum += static_cast<float>(val);
                for (uint32_t p = 0; p < 4; ++p) {
                    plane[p] |= ((q >> p) & 1U) << e;
                }
            }
            for (uint32_t p = 0; p < 4; ++p) {
                qc[p * l.plane_bytes + b] = static_cast<uint8_t>(plane[p]);
            }
        }
        for (int off = 32; off > 0; off >>= 1) {
            qsum += __shfl_xor(qsum, off);
        }
        if (lane == 0) {
            store_f32(qc + l.q_offset_lb, lb);
            store_f32(qc + l.q_offset_delta, delta);
            store_f32(qc + l.q_offset_sum, qsum);
        }
    } else {
        for (uint32_t d = lane; d < dim; d += kWave) {
            store_f32(qc + 4 * d, t[d] / norm);
        }
    }
    if (lane == 0) {
        store_f32(qc + l.q_offset_norm, norm);
        if (l.has_raw_norm) {
            store_f32(qc + l.q_offset_raw_norm, raw_norm);
        }
    }
}

int
squ_encode_launch(const float* x, uint64_t n, uint32_t dim, int bits, int metric, const float* bounds, uint8_t* codes,
                  hipStream_t st, float* norm_scratch) {
    if (n == 0) {
        return 0;
    }
    int kind = bits == 4 ? VSAG_AMD_KIND_SQ4_UNIFORM : VSAG_AMD_KIND_SQ8_UNIFORM;
    uint32_t code_size = static_cast<uint32_t>(vsag_amd_code_size(kind, metric, dim, 0));
    uint32_t payload = bits == 4 ? (dim + 1) / 2 : dim;
    bool norm = metric == VSAG_AMD_METRIC_L2 || (bits == 4 && metric == VSAG_AMD_METRIC_COSINE);
    uint32_t align = norm ? 8 : 4;
    uint32_t off = static_cast<uint32_t>(round_up(payload, align));
    uint32_t off_norm = off;
    uint32_t off_sum = off + (norm ? 8 : 0);
    uint32_t off_codes_sum = off_sum + align;
    // Cosine needs a float per row; a caller that must not allocate brings them (norm_scratch, n floats).
    float* norms = nullptr;
    if (metric == VSAG_AMD_METRIC_COSINE) {
        norms = norm_scratch;
        if (norms == nullptr) {
            VA_HIP(hipMallocAsync(reinterpret_cast<void**>(&norms), n * 4, st));
        }
        hipLaunchKernelGGL(row_norm_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, x, n, dim,
                           norms);
    }
    hipLaunchKernelGGL(squ_encode_kernel, dim3(static_cast<uint32_t>(div_up(n, 4))), dim3(256), 0, st, x, n, dim, bits,
                       metric, bounds, norms, code_size, payload, off_norm, off_sum, off_codes_sum, codes);
    VA_HIP(hipGetLastError());
    if (norms != nullptr && norms != norm_scratch) {
        VA_HIP(hipFreeAsync(norms, st));
    }
    return 0;
}

// Rotates rows in slabs so that the temporary stays bounded, then runs `finish` on each slab.  The temporary
// (min(n, kRotateSlabRows) x dim floats) is `scratch` when the caller brings one, else allocated on the stream.
template <typename Finish>
static int
rabitq_rotate_slabs(const float* x, uint64_t n, uint32_t dim, const float* rot, hipStream_t st, float* scratch,
                    Finish finish) {
    const uint64_t slab = kRotateSlabRows;
    uint64_t rows = n < slab ? n : slab;
    float* tmp = scratch;
    if (tmp == nullptr) {
        VA_HIP(hipMallocAsync(reinterpret_cast<void**>(&tmp), rows * dim * 4, st));
    }
    int rc = 0;
    for (uint64_t s = 0; s < n && rc == 0; s += slab) {
        uint64_t m = n - s < slab ? n - s : slab;
        rc = gemm_nt_seq(x + s * dim, rot, tmp, m, dim, dim, st);
        if (rc == 0) {
            rc = finish(s, m, tmp);
        }
    }
    if (tmp != scratch) {
        hipError_t e = hipFreeAsync(tmp, st);
        if (rc == 0 && e != hipSuccess) {
            return fail(VSAG_AMD_INTERNAL_ERROR, "hipFreeAsync failed: %s", hipGetErrorString(e));
        }
    }
    return rc;
}

int
rabitq_process_query_launch(const float* q, uint64_t nq, uint32_t dim, const float* rot, const float* centroid,
                            int metric, int query_bits, uint8_t* qcodes, hipStream_t st, float* scratch) {
    if (nq == 0) {
        return 0;
    }
    uint64_t qsize = rabitq_query_code_size(dim, metric, query_bits);
    return rabitq_rotate_slabs(q, nq, dim, rot, st, scratch, [&](uint64_t s, uint64_t m, const float* rotated) {
        const size_t lds = static_cast<size_t>(dim) * 4 * (rabitq_layout(dim, metric, query_bits).has_raw_norm ? 2 : 1);
        if (lds <= 48 * 1024) {
            hipLaunchKernelGGL(rabitq_finish_query_wave_kernel, dim3(static_cast<uint32_t>(m)), dim3(64), lds, st,
                               q + s * dim, rotated, m, dim, centroid, metric, query_bits, qcodes + s * qsize);
        } else {
            hipLaunchKernelGGL(rabitq_finish_query_kernel, dim3(static_cast<uint32_t>(div_up(m, 64))), dim3(64), 0, st,
                               q + s * dim, rotated, m, dim, centroid, metric, query_bits, qcodes + s * qsize);
        }
        VA_HIP(hipGetLastError());
        return 0;
    });
}

// ------------------------------------------------------------------ scalar-quantization trainer
// Sample gather (scalar_quantization_trainer.cpp:125-146): row j of the sample is row (j * step) % n,
// written transposed (sample_t[d][j]) so that the per-dimension selection reads contiguously.
__global__ void __launch_bounds__(256)
sq_sample_kernel(const float* x, uint64_t n, uint32_t dim, uint64_t step, uint64_t sample_count, const float* norms,
                 float* sample_t) {
    uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint64_t j = gid / dim;
    uint32_t d = static_cast<uint32_t>(gid % dim);
    if (j >= sample_count) {
        return;
    }
    uint64_t idx = (j * step) % n;
    float v = x[idx * dim + d];
    if (norms != nullptr) {
        v = v / norms[idx];
    }
    sample_t[static_cast<uint64_t>(d) * sample_count + j] = v;
}

// k-th smallest (1-based) of vals[0,count) by an 8-bit radix descent over order-preserving keys.
// One workgroup per call site; hist is a 256-entry LDS array.
__device__ inline float
block_kth_smallest(const float* vals, uint64_t count, uint64_t kth, uint32_t* hist, uint32_t* shared) {
    uint32_t prefix = 0, mask = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (uint32_t i = threadIdx.x; i < 256; i += blockDim.x) {
            hist[i] = 0;
        }
        __syncthreads();
        for (uint64_t i = threadIdx.x; i < count; i += blockDim.x) {
            uint32_t key = float_to_ordered(vals[i]);
            if ((key & mask) == prefix) {
                atomicAdd(&hist[(key >> shift) & 0xff], 1U);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            uint64_t acc = 0;
            uint32_t bin = 0;
            for (; bin < 256; ++bin) {
                if (acc + hist[bin] >= kth) {
                    break;
                }
                acc += hist[bin];
            }
            shared[0] = bin;
            shared[1] = static_cast<uint32_t>(acc);
        }
        __syncthreads();
        prefix |= shared[0] << shift;
        mask |= 0xffU << shift;
        kth -= shared[1];
        __syncthreads();
    }
    return ordered_to_float(prefix);
}

// trunc_bound_train / classic_train (scalar_quantization_trainer.cpp:72-122): the bounded heaps keep the
// ignore_count largest and smallest sample values of a dimension; their tops are the ignore_count-th
// largest and smallest.  CLASSIC is the same with ignore_count = 1.  Writes lower bound and diff.
__global__ void __launch_bounds__(256)
sq_bounds_kernel(const float* sample_t, uint64_t count, uint32_t dim, uint64_t ignore_count, float* lb, float* diff,
                 float* upper_out, float* lower_out) {
    __shared__ uint32_t hist[256];
    __shared__ uint32_t shared[2];
    uint32_t d = blockIdx.x;
    const float* col = sample_t + static_cast<uint64_t>(d) * count;
    uint64_t k = ignore_count < count ? ignore_count : count;
    float lower = block_kth_smallest(col, count, k, hist, shared);
    float upper = block_kth_smallest(col, count, count - k + 1, hist, shared);
    if (threadIdx.x == 0) {
        if (lb != nullptr) {
            lb[d] = lower;
            diff[d] = upper - lower;
        }
        if (upper_out != nullptr) {
            upper_out[d] = upper;
            lower_out[d] = lower;
        }
    }
}

// TrainUniform (scalar_quantization_trainer.cpp:47-70): CLASSIC -> max of uppers / min of lowers;
// TRUNC_BOUND -> min of uppers / max of lowers, swapped when inverted.  out = {lb, diff}.
__global__ void
sq_uniform_reduce_kernel(const float* upper, const float* lower, uint32_t dim, int mode, float* out) {
    if (threadIdx.x != 0 || blockIdx.x != 0) {
        return;
    }
    float ub = upper[0], lb = lower[0];
    for (uint32_t d = 1; d < dim; ++d) {
        if (mode == VSAG_AMD_SQ_TRAIN_CLASSIC) {
            ub = fmaxf(ub, upper[d]);
            lb = fminf(lb, lower[d]);
        } else {
            ub = fminf(ub, upper[d]);
            lb = fmaxf(lb, lower[d]);
        }
    }
    if (mode != VSAG_AMD_SQ_TRAIN_CLASSIC && lb > ub) {
        float t = lb;
        lb = ub;
        ub = t;
    }
    out[0] = lb;
    out[1] = ub - lb;
}

struct TrainPlan {
    uint64_t sample_count, step, ignore_count;
};

static TrainPlan
train_plan(uint64_t n, int bits, int mode, float trunc_rate, uint64_t max_sample) {
    TrainPlan p{};
    if (max_sample == 0) {
        max_sample = 100000;
    }
    p.step = 2147483647ULL % n;
    p.sample_count = max_sample;
    if (n <= max_sample) {
        p.step = 1;
        p.sample_count = n;
    }
    if (mode == VSAG_AMD_SQ_TRAIN_CLASSIC) {
        p.ignore_count = 1;
    } else {
        double rate = bits == 4 ? static_cast<double>(trunc_rate) : 0.001;
        auto ic = static_cast<uint64_t>(static_cast<double>(p.sample_count - 1) * rate);
        p.ignore_count = ic < 1 ? 1 : ic;
    }
    return p;
}

static int
sq_train_common(const float* x, uint64_t n, uint32_t dim, int bits, int metric, int mode, float trunc_rate,
                uint64_t max_sample, float* lb, float* diff, float* uniform_out, void* ws, size_t ws_bytes,
                hipStream_t st) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(x != nullptr && n >= 1, "sq_train needs at least one row");
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(bits == 4 || bits == 8, "bits must be 4 or 8, got %d", bits);
    VA_CHECK_ARG(mode == VSAG_AMD_SQ_TRAIN_CLASSIC || mode == VSAG_AMD_SQ_TRAIN_TRUNC_BOUND, "unknown train mode %d",
                 mode);
    TrainPlan p = train_plan(n, bits, mode, trunc_rate, max_sample);
    Carver c(ws, ws_bytes);
    float* sample_t = c.take<float>(p.sample_count * dim);
    float* norms = c.take<float>(metric == VSAG_AMD_METRIC_COSINE ? n : 0);
    float* upper = c.take<float>(dim);
    float* lower = c.take<float>(dim);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, ws_bytes);
    if (metric == VSAG_AMD_METRIC_COSINE) {
        hipLaunchKernelGGL(row_norm_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, x, n, dim,
                           norms);
    } else {
        norms = nullptr;
    }
    hipLaunchKernelGGL(sq_sample_kernel, dim3(static_cast<uint32_t>(div_up(p.sample_count * dim, 256))), dim3(256), 0,
                       st, x, n, dim, p.step, p.sample_count, norms, sample_t);
    hipLaunchKernelGGL(sq_bounds_kernel, dim3(dim), dim3(256), 0, st, sample_t, p.sample_count, dim, p.ignore_count,
                       lb, diff, upper, lower);
    if (uniform_out != nullptr) {
        hipLaunchKernelGGL(sq_uniform_reduce_kernel, dim3(1), dim3(64), 0, st, upper, lower, dim, mode, uniform_out);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_sq_train_workspace_bytes(uint64_t n, uint32_t dim, uint64_t max_sample) {
    if (n == 0) {
        return 0;
    }
    TrainPlan p = train_plan(n, 8, VSAG_AMD_SQ_TRAIN_TRUNC_BOUND, 0.05F, max_sample);
    return round_up(p.sample_count * dim * 4, 256) + round_up(n * 4, 256) + 2 * round_up(dim * 4ull, 256) + 256;
}

extern "C" int
vsag_amd_sq_train(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric, int mode, float trunc_rate,
                  uint64_t max_sample, float* lower_bound_dev, float* diff_dev, void* workspace_dev,
                  size_t workspace_bytes, void* stream) {
    VA_CHECK_ARG(lower_bound_dev && diff_dev, "null output");
    return sq_train_common(x_dev, n, dim, bits, metric, mode, trunc_rate, max_sample, lower_bound_dev, diff_dev,
                           nullptr, workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int
vsag_amd_sq_train_uniform(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric, int mode,
                          float trunc_rate, uint64_t max_sample, float* out_dev, void* workspace_dev,
                          size_t workspace_bytes, void* stream) {
    VA_CHECK_ARG(out_dev, "null output");
    return sq_train_common(x_dev, n, dim, bits, metric, mode, trunc_rate, max_sample, nullptr, nullptr, out_dev,
                           workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int
vsag_amd_sq_encode(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric, const float* lower_bound_dev,
                   const float* diff_dev, uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(bits == 4 || bits == 8, "bits must be 4 or 8, got %d", bits);
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(x_dev && lower_bound_dev && diff_dev && codes_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t code_size = (dim * bits + 7) / 8;
    float* norms = nullptr;
    if (metric == VSAG_AMD_METRIC_COSINE) {
        VA_HIP(hipMallocAsync(reinterpret_cast<void**>(&norms), n * 4, st));
        hipLaunchKernelGGL(row_norm_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, x_dev, n,
                           dim, norms);
    }
    uint64_t threads = n * code_size;
    VA_CHECK_ARG(div_up(threads, 256) < (1ull << 31), "too many rows for one encode call");
    hipLaunchKernelGGL(sq_encode_kernel, dim3(static_cast<uint32_t>(div_up(threads, 256))), dim3(256), 0, st, x_dev, n,
                       dim, bits, lower_bound_dev, diff_dev, norms, code_size, codes_dev);
    VA_HIP(hipGetLastError());
    if (norms != nullptr) {
        VA_HIP(hipFreeAsync(norms, st));
    }
    return 0;
}

extern "C" int
vsag_amd_squ_encode(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric, const float* bounds_dev,
                    uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(bits == 4 || bits == 8, "bits must be 4 or 8, got %d", bits);
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(n == 0 || (x_dev && bounds_dev && codes_dev), "null pointer");
    return squ_encode_launch(x_dev, n, dim, bits, metric, bounds_dev, codes_dev, static_cast<hipStream_t>(stream),
                             nullptr);
}

extern "C" int
vsag_amd_rabitq_train(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev, float* centroid_dev,
                      void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(x_dev && rotation_dev && centroid_dev && n >= 1, "null pointer or empty data");
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    hipStream_t st = static_cast<hipStream_t>(stream);
    float* mean = nullptr;
    VA_HIP(hipMallocAsync(reinterpret_cast<void**>(&mean), dim * 4, st));
    hipLaunchKernelGGL(column_mean_seq_kernel, dim3((dim + kMeanCols - 1) / kMeanCols), dim3(1024), 0, st, x_dev, n, dim,
                       mean);
    int rc = gemm_nt_seq(mean, rotation_dev, centroid_dev, 1, dim, dim, st);
    VA_HIP(hipFreeAsync(mean, st));
    return rc;
}

extern "C" int
vsag_amd_rabitq_encode(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                       const float* centroid_dev, int metric, int query_bits, uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(query_bits == 4 || query_bits == 32, "query_bits must be 4 or 32, got %d", query_bits);
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(x_dev && rotation_dev && centroid_dev && codes_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint64_t csize = rabitq_code_size(dim, metric, query_bits);
    return rabitq_rotate_slabs(x_dev, n, dim, rotation_dev, st, nullptr, [&](uint64_t s, uint64_t m, const float* rotated) {
        hipLaunchKernelGGL(rabitq_finish_encode_kernel, dim3(static_cast<uint32_t>(div_up(m, 64))), dim3(64), 0, st,
                           x_dev + s * dim, rotated, m, dim, centroid_dev, metric, query_bits, codes_dev + s * csize);
        VA_HIP(hipGetLastError());
        return 0;
    });
}

// FhtKacRotator (impl/transform/fht_kac_rotate_transformer.cpp:64-96, rabitq_use_fht) as the dense matrix the rabitq
// entry points take: y = R x with R[i][j] = Transform(e_j)[i].  The rotator is a product of sign flips, Hadamard
// butterflies on a power-of-two block, Kac walks and scalings, all of them row operations on the matrix of the
// transformed basis vectors (one column per basis vector), which starts as the identity.  Host memory on both sides.
extern "C" int
vsag_amd_fht_kac_matrix(const uint8_t* flip, uint32_t dim, float* rotation) {
    VA_CHECK_ARG(flip != nullptr && rotation != nullptr, "null pointer");
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    const size_t d = dim;
    const size_t flip_bytes = (d + 7) / 8;
    size_t block = 1;  // the largest power of two within dim
    while (block * 2 <= d) {
        block *= 2;
    }
    const float scale = 1.0F / std::sqrt(static_cast<float>(block));
    std::fill(rotation, rotation + d * d, 0.0F);
    for (size_t i = 0; i < d; ++i) {
        rotation[i * d + i] = 1.0F;
    }
    auto row = [&](size_t i) { return rotation + i * d; };
    auto flip_rows = [&](int round) {
        const uint8_t* f = flip + static_cast<size_t>(round) * flip_bytes;
        for (size_t i = 0; i < d; ++i) {
            if ((f[i >> 3] >> (i & 7)) & 1) {
                float* r = row(i);
                for (size_t j = 0; j < d; ++j) {
                    r[j] = -r[j];
                }
            }
        }
    };
    auto pair_rows = [&](size_t a, size_t b) {  // (a, b) <- (a + b, a - b)
        float* ra = row(a);
        float* rb = row(b);
        for (size_t j = 0; j < d; ++j) {
            const float x = ra[j], y = rb[j];
            ra[j] = x + y;
            rb[j] = x - y;
        }
    };
    auto scale_rows = [&](size_t first, size_t count, float v) {
        for (size_t i = first; i < first + count; ++i) {
            float* r = row(i);
            for (size_t j = 0; j < d; ++j) {
                r[j] *= v;
            }
        }
    };
    auto hadamard = [&](size_t first) {
        for (size_t step = 1; step < block; step *= 2) {
            for (size_t i = 0; i < block; i += 2 * step) {
                for (size_t j = 0; j < step; ++j) {
                    pair_rows(first + i + j, first + i + j + step);
                }
            }
        }
        scale_rows(first, block, scale);
    };
    auto kac_walk = [&]() {
        const size_t half = d / 2, offset = half + d % 2;
        for (size_t i = 0; i < half; ++i) {
            pair_rows(i, i + offset);
        }
        if (d % 2 != 0) {
            scale_rows(half, 1, std::sqrt(2.0F));
        }
    };
    if (block == d) {
        for (int round = 0; round < 4; ++round) {
            flip_rows(round);
            hadamard(0);
        }
        return 0;
    }
    for (int round = 0; round < 4; round += 2) {
        flip_rows(round);
        hadamard(0);
        kac_walk();
        flip_rows(round + 1);
        hadamard(d - block);
        kac_walk();
    }
    scale_rows(0, d, 0.25F);  // four Kac walks, each of which doubles the squared length
    return 0;
}

// RaBitQuantizer::DecodeOneImpl (rabitq_quantizer.cpp:871-899), 1-bit codes: y = (+-1 / sqrt(d)) * norm + centroid
// per dimension (InverseNormalizeWithCentroid, simd/kernels/normalize.h:88-119), x = R^T y.  A workgroup per code, a
// thread per output dimension, the rows of R summed in order.
__global__ void __launch_bounds__(256)
rabitq_decode_kernel(const uint8_t* codes, uint32_t dim, const float* rot, const float* centroid, uint32_t code_size,
                     uint32_t offset_norm, float* out) {
    const uint64_t i = blockIdx.x;
    const uint8_t* c = codes + i * code_size;
    const float norm = load_f32(c + offset_norm);
    const float inv_sqrt_d = 1.0F / sqrtf(static_cast<float>(dim));
    for (uint32_t j = threadIdx.x; j < dim; j += blockDim.x) {
        float acc = 0.0F;
        for (uint32_t r = 0; r < dim; ++r) {
            const bool bit = ((c[r >> 3] >> (r & 7)) & 1) != 0;
            const float y = (bit ? inv_sqrt_d : -inv_sqrt_d) * norm + centroid[r];
            acc += rot[static_cast<uint64_t>(r) * dim + j] * y;
        }
        out[i * dim + j] = acc;
    }
}

extern "C" int
vsag_amd_rabitq_decode(const uint8_t* codes_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                       const float* centroid_dev, int metric, int bits_word, float* out_dev, void* stream) {
    VA_TRY(ensure_init());
    const int query_bits = bits_word & 255;
    VA_CHECK_ARG(query_bits == 4 || query_bits == 32, "query_bits must be 4 or 32, got %d", query_bits);
    VA_CHECK_ARG((bits_word >> 8) <= 1, "only 1-bit codes decode (RaBitQuantizer::DecodeOneImpl returns false for the others)");
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev && rotation_dev && centroid_dev && out_dev, "null pointer");
    VA_CHECK_ARG(n < (1ull << 31), "n must be below 2^31");
    const RabitqLayout l = rabitq_layout(dim, metric, query_bits);
    hipLaunchKernelGGL(rabitq_decode_kernel, dim3(static_cast<uint32_t>(n)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       codes_dev, dim, rotation_dev, centroid_dev, l.code_size, l.offset_norm, out_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_rabitq_encode_multibit(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                                const float* centroid_dev, int metric, int bits_word, int fast_encode,
                                uint32_t fast_encode_rounds, uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    const int base_bits = bits_word >> 8;
    VA_CHECK_ARG((bits_word & 255) == 32, "multi-bit base codes need fp32 queries (query bits 32), got %d", bits_word & 255);
    VA_CHECK_ARG(base_bits >= 2 && base_bits <= 8, "base bits must be in [2, 8], got %d", base_bits);
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(!fast_encode || (fast_encode_rounds >= 1 && fast_encode_rounds <= 32),
                 "fast_encode_rabitq_rounds must be in [1, 32], but got %u", fast_encode_rounds);
    VA_CHECK_ARG(fast_encode || dim <= 3072, "the exhaustive encoder supports at most 3072 dimensions, got %u", dim);
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(x_dev && rotation_dev && centroid_dev && codes_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint64_t csize = rabitq_code_size(dim, metric, bits_word);
    const uint64_t rows = n < kRotateSlabRows ? n : kRotateSlabRows;
    uint8_t* scalar = nullptr;
    float* norm_code = nullptr;
    VA_HIP(hipMallocAsync(reinterpret_cast<void**>(&scalar), rows * dim, st));
    hipError_t e = hipMallocAsync(reinterpret_cast<void**>(&norm_code), rows * 4, st);
    if (e != hipSuccess) {
        (void)hipFreeAsync(scalar, st);
        return fail(VSAG_AMD_NO_ENOUGH_MEMORY, "hipMallocAsync failed: %s", hipGetErrorString(e));
    }
    int rc = rabitq_rotate_slabs(x_dev, n, dim, rotation_dev, st, nullptr, [&](uint64_t s, uint64_t m, const float* rotated) {
        if (fast_encode) {
            hipLaunchKernelGGL(rabitq_fast_encode_kernel, dim3(static_cast<uint32_t>(div_up(m, 64))), dim3(64), 0, st,
                               rotated, m, dim, centroid_dev, static_cast<uint32_t>(base_bits), fast_encode_rounds, scalar,
                               norm_code);
        } else {
            const size_t lds = static_cast<size_t>(dim) * 16;
            hipLaunchKernelGGL(rabitq_extend_encode_kernel, dim3(static_cast<uint32_t>(m)), dim3(64), lds, st, rotated, m,
                               dim, centroid_dev, static_cast<uint32_t>(base_bits), scalar, norm_code);
        }
        VA_HIP(hipGetLastError());
        hipLaunchKernelGGL(rabitq_multibit_finish_kernel, dim3(static_cast<uint32_t>(div_up(m, 64))), dim3(64), 0, st,
                           x_dev + s * dim, rotated, m, dim, centroid_dev, metric, bits_word, scalar, norm_code,
                           codes_dev + s * csize);
        VA_HIP(hipGetLastError());
        return 0;
    });
    (void)hipFreeAsync(scalar, st);
    (void)hipFreeAsync(norm_code, st);
    return rc;
}

extern "C" uint64_t
vsag_amd_rabitq_query_code_size(uint32_t dim, int metric, int query_bits) {
    return rabitq_query_code_size(dim, metric, query_bits);
}

extern "C" int
vsag_amd_rabitq_process_query(const float* q_dev, uint64_t nq, uint32_t dim, const float* rotation_dev,
                              const float* centroid_dev, int metric, int query_bits, uint8_t* qcodes_dev,
                              void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG((query_bits & 255) == 4 || (query_bits & 255) == 32, "query_bits must be 4 or 32, got %d",
                 query_bits & 255);
    VA_CHECK_ARG((query_bits >> 8) == 0 || ((query_bits & 255) == 32 && (query_bits >> 8) <= 8),
                 "multi-bit base codes (%d bits) need fp32 queries and at most 8 bits", query_bits >> 8);
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(nq == 0 || (q_dev && rotation_dev && centroid_dev && qcodes_dev), "null pointer");
    return rabitq_process_query_launch(q_dev, nq, dim, rotation_dev, centroid_dev, metric, query_bits, qcodes_dev,
                                       static_cast<hipStream_t>(stream), nullptr);
}
