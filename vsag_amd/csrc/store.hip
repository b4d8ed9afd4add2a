// Code stores: creation, growth, and re-tiling of reference-layout codes into the wave64 tile layout
// (the device-side counterpart of FlattenDataCell::BatchInsertVector, src/datacell/flatten_datacell.h:279-314,
// and of BucketDataCell::InsertVector, src/datacell/bucket_datacell.h:670-709).
#include <hipcub/hipcub.hpp>

#include <cmath>
#include <new>

#include "store.h"

namespace vsag_amd {

uint64_t rabitq_code_size(uint32_t dim, int metric, int query_bits);

// dst_slot[i] = tile slot (tile * 64 + lane) of source code i; src_index[i] = row of the source code.
// One thread per (code, granule): gathers up to 16 payload bytes and writes one uint4; the thread of
// granule 0 also moves the per-code metadata words.
struct RetileArgs {
    const uint8_t* codes;
    uint64_t n;
    uint32_t code_size;
    uint32_t payload_bytes;
    uint32_t plane_bytes;     // source bytes of one plane of the payload ...
    uint32_t plane_granules;  // ... which fill this many granules (zero padded)
    uint32_t G;
    uint32_t nmeta;
    uint32_t meta_offset[4];
    uint32_t meta_is_u64;
    uint4* tiles;
    uint32_t* meta;
    uint64_t meta_stride;
    uint64_t first_slot;          // flat append: slot of source code 0
    const uint32_t* src_index;    // list form: sorted position -> source row (may be null)
    const uint32_t* dst_slot;     // list form: sorted position -> tile slot (may be null)
    uint32_t* ids;                // list form: inner id per slot
    uint32_t id_base;             // list form: inner id of source row 0
    uint32_t* slot_of_id;         // list form: slot per inner id
    const float* bias_src;        // list form: per source row residual bias (may be null)
    float* bias_dst;              // list form: per slot
    int normalize;                // fp32 + cosine: store x / ||x||
    uint32_t dim;
};

__global__ void __launch_bounds__(256)
retile_kernel(RetileArgs a) {
    uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint64_t i = gid / a.G;
    uint32_t j = static_cast<uint32_t>(gid % a.G);
    if (i >= a.n) {
        return;
    }
    uint64_t row = a.src_index ? a.src_index[i] : i;
    uint64_t slot = a.dst_slot ? a.dst_slot[i] : a.first_slot + i;
    const uint8_t* src = a.codes + row * a.code_size;
    uint32_t w[4] = {0, 0, 0, 0};
    if (a.normalize) {
        const float* x = reinterpret_cast<const float*>(src);
        float s = 0.0F;
        for (uint32_t d = 0; d < a.dim; ++d) {
            s = fmaf(x[d], x[d], s);
        }
        float norm = sqrtf(s);
        if (norm == 0.0F) {
            norm = 1.0F;  // DivScalarImpl (src/simd/kernels/scalar_op.h:40-42): a zero norm divides by 1
        }
        for (uint32_t e = 0; e < 4; ++e) {
            uint32_t d = 4 * j + e;
            if (d < a.dim) {
                w[e] = __float_as_uint(x[d] / norm);
            }
        }
    } else {
        const uint32_t plane = j / a.plane_granules;
        const uint8_t* run = src + plane * a.plane_bytes;
        for (uint32_t b = 0; b < 16; ++b) {
            uint32_t off = 16 * (j - plane * a.plane_granules) + b;
            if (off < a.plane_bytes) {
                w[b >> 2] |= static_cast<uint32_t>(run[off]) << (8 * (b & 3));
            }
        }
    }
    uint64_t tile = slot / kWave;
    uint32_t lane = static_cast<uint32_t>(slot % kWave);
    a.tiles[(tile * a.G + j) * kWave + lane] = make_uint4(w[0], w[1], w[2], w[3]);
    if (j == 0) {
        for (uint32_t m = 0; m < a.nmeta; ++m) {
            if (a.meta_offset[m] == kMetaPayloadSum) {
                uint32_t sum = 0;
                for (uint32_t b = 0; b < a.payload_bytes; ++b) {
                    sum += src[b];
                }
                a.meta[m * a.meta_stride + slot] = sum;
                continue;
            }
            const uint8_t* p = src + a.meta_offset[m];
            uint32_t word;
            if ((a.meta_is_u64 >> m) & 1) {
                uint64_t v = 0;
                for (int b = 0; b < 8; ++b) {
                    v |= static_cast<uint64_t>(p[b]) << (8 * b);
                }
                word = __float_as_uint(static_cast<float>(v));
            } else {
                word = 0;
                for (int b = 0; b < 4; ++b) {
                    word |= static_cast<uint32_t>(p[b]) << (8 * b);
                }
            }
            a.meta[m * a.meta_stride + slot] = word;
        }
        if (a.ids != nullptr) {
            const uint32_t id = a.id_base + static_cast<uint32_t>(row);
            a.ids[slot] = id;
            a.slot_of_id[id] = static_cast<uint32_t>(slot);
            if (a.bias_dst != nullptr) {
                a.bias_dst[slot] = a.bias_src != nullptr ? a.bias_src[row] : 0.0F;
            }
        }
    }
}

__global__ void
fill_u32_kernel(uint32_t* p, uint32_t v, uint64_t n) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

__global__ void
scale_table_kernel(const float* lb, const float* diff, uint32_t dim, uint32_t dpad, float levels, float* scale,
                   float* lb_out, float* diff_out) {
    uint32_t d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d < dpad) {
        scale[d] = d < dim ? diff[d] / levels : 0.0F;
        lb_out[d] = d < dim ? lb[d] : 0.0F;
        diff_out[d] = d < dim ? diff[d] : 0.0F;
    }
}

__global__ void
histogram_kernel(const int32_t* labels, uint64_t n, uint32_t nlist, uint32_t* counts, uint32_t* bad) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        int32_t l = labels[i];
        if (l < 0 || static_cast<uint32_t>(l) >= nlist) {
            atomicAdd(bad, 1U);
        } else {
            atomicAdd(&counts[l], 1U);
        }
    }
}

__global__ void
iota_kernel(uint32_t* p, uint64_t n) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = static_cast<uint32_t>(i);
    }
}

// sorted position p (the new codes ordered by label, stable) -> tile slot: slot_base[l] + p, slot_base[l] = first free
// slot of list l minus the position of the list's first new code (modulo 2^32).
__global__ void
list_slot_kernel(const int32_t* sorted_labels, uint64_t n, const uint32_t* slot_base, uint32_t* dst_slot) {
    uint64_t p = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p < n) {
        dst_slot[p] = slot_base[static_cast<uint32_t>(sorted_labels[p])] + static_cast<uint32_t>(p);
    }
}

// Moves the used tiles of every list to the list's new place (one workgroup per old tile).
struct RelocateArgs {
    const uint4* old_tiles;
    uint4* new_tiles;
    uint32_t G;
    const uint32_t* old_lt;     // 2 * nlist (first tile, end of used tiles)
    const uint32_t* new_begin;  // nlist
    uint32_t nlist;
    const uint32_t* old_meta;
    uint32_t* new_meta;
    uint32_t nmeta;
    uint64_t old_stride, new_stride;
    const uint32_t* old_ids;
    uint32_t* new_ids;
    uint32_t* slot_of_id;
    const float* old_bias;  // may be null
    float* new_bias;
};

__global__ void __launch_bounds__(256)
relocate_tiles_kernel(RelocateArgs a) {
    __shared__ uint32_t target;
    const uint32_t t = blockIdx.x;
    if (threadIdx.x == 0) {
        // the last list whose first tile is at or before t (first tiles ascend)
        uint32_t lo = 0, hi = a.nlist;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (a.old_lt[2 * mid] <= t) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        target = t >= a.old_lt[2 * lo] && t < a.old_lt[2 * lo + 1] ? a.new_begin[lo] + (t - a.old_lt[2 * lo]) : 0xFFFFFFFFU;
    }
    __syncthreads();
    const uint32_t nt = target;
    if (nt == 0xFFFFFFFFU) {
        return;  // room behind a list, not in use
    }
    for (uint32_t i = threadIdx.x; i < a.G * kWave; i += blockDim.x) {
        a.new_tiles[static_cast<uint64_t>(nt) * a.G * kWave + i] = a.old_tiles[static_cast<uint64_t>(t) * a.G * kWave + i];
    }
    if (threadIdx.x < kWave) {
        const uint64_t os = static_cast<uint64_t>(t) * kWave + threadIdx.x, ns = static_cast<uint64_t>(nt) * kWave + threadIdx.x;
        for (uint32_t m = 0; m < a.nmeta; ++m) {
            a.new_meta[m * a.new_stride + ns] = a.old_meta[m * a.old_stride + os];
        }
        const uint32_t id = a.old_ids[os];
        a.new_ids[ns] = id;
        if (id != VSAG_AMD_INVALID_ID) {
            a.slot_of_id[id] = static_cast<uint32_t>(ns);
        }
        if (a.new_bias != nullptr) {
            a.new_bias[ns] = a.old_bias != nullptr ? a.old_bias[os] : 0.0F;
        }
    }
}

// Stores whose large batches are pre-selected on the matrix cores and rescored (prefilter.hip).
static bool
keeps_rows(const vsag_amd_store* s) {
    // Not fp32 stores: the copy would double the largest of all stores for the smallest gain.
    return (s->pf_ymax != nullptr && s->kind != VSAG_AMD_KIND_FP32) ||
           (s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4);
}

// rows[slot][j] = granule j of the code in `slot`, from the tiles; with row_granules = G + 1 the last granule of a row
// holds the code's metadata words (zero beyond nmeta).
__global__ void __launch_bounds__(256)
rows_from_tiles_kernel(const uint4* tiles, uint32_t G, uint32_t row_granules, const uint32_t* meta, uint64_t meta_stride,
                       uint32_t nmeta, uint64_t first_slot, uint64_t count, uint4* rows) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count * row_granules) {
        return;
    }
    const uint64_t slot = first_slot + i / row_granules;
    const uint32_t j = static_cast<uint32_t>(i % row_granules);
    if (j < G) {
        rows[slot * row_granules + j] = tiles[((slot / kWave) * G + j) * kWave + slot % kWave];
    } else {
        uint32_t w[4] = {0, 0, 0, 0};
        for (uint32_t m = 0; m < nmeta && m < 4; ++m) {
            w[m] = meta[m * meta_stride + slot];
        }
        rows[slot * row_granules + j] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// Stores whose code bits are kept as fp4 operands as well (prefilter_rb.hip).
static bool
keeps_f4(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_RABITQ && s->query_bits == 4 && s->base_bits == 1 && s->G <= kRbMaxG &&
           (s->metric == VSAG_AMD_METRIC_L2 || s->metric == VSAG_AMD_METRIC_IP);
}

__device__ inline uint32_t
f4_order(uint32_t w) {
    // bit 8 v + j -> bit 4 j + v
    uint32_t out = 0;
#pragma unroll
    for (uint32_t v = 0; v < 4; ++v) {
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            out |= ((w >> (8 * v + j)) & 1U) << (4 * j + v);
        }
    }
    return out;
}

// f4tiles of tiles [first_tile, first_tile + ntiles) from the tiles; a thread per (tile, granule, lane).
__global__ void __launch_bounds__(256)
f4_from_tiles_kernel(const uint4* tiles, uint32_t G, uint64_t first_tile, uint64_t ntiles, uint4* f4tiles) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= ntiles * G * kWave) {
        return;
    }
    const uint64_t at = first_tile * G * kWave + i;  // (tile G + g) 64 + lane
    const uint32_t lane = static_cast<uint32_t>(at % kWave);
    const uint64_t granule = at - lane;
    const uint32_t h = lane >> 5, r = lane & 31;
    const uint4 lo = tiles[granule + r], hi = tiles[granule + 32 + r];
    uint4 out;
    out.x = f4_order(h == 0 ? lo.x : lo.y);
    out.y = f4_order(h == 0 ? lo.z : lo.w);
    out.z = f4_order(h == 0 ? hi.x : hi.y);
    out.w = f4_order(h == 0 ? hi.z : hi.w);
    f4tiles[at] = out;
}

// f4const of slots [first_slot, first_slot + count).  With err the error factor, norm and raw the norms of a code and
// S its sum field: A = err / (2 norm), B = (norm^2 [- raw^2]) A, S.  Codes the derivation of the pass does not cover
// (zero norm, non-positive error factor, zero raw norm, factors so large that the fp32 threshold would lose its margin,
// a sum field that is not the number of set bits -- the matrix cores count the bits themselves) stand outside.
__global__ void __launch_bounds__(256)
f4_const_kernel(const uint4* tiles, uint32_t G, const uint32_t* meta, uint64_t meta_stride, int is_l2, const uint32_t* ids,
                uint64_t n, uint64_t first_slot, uint64_t count, float4* f4const) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count) {
        return;
    }
    const uint64_t slot = first_slot + i;
    const uint4* code = tiles + (slot / kWave) * G * kWave + slot % kWave;
    uint32_t bits = 0;
    for (uint32_t g = 0; g < G; ++g) {
        const uint4 v = code[static_cast<uint64_t>(g) * kWave];
        bits += __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
    }
    const float bn = __uint_as_float(meta[slot]);
    float berr = __uint_as_float(meta[meta_stride + slot]);
    const float bsum = __uint_as_float(meta[2 * meta_stride + slot]);
    const float braw = is_l2 ? 0.0F : __uint_as_float(meta[3 * meta_stride + slot]);
    if (fabsf(berr) < 1e-5F) {
        berr = berr >= 0 ? 1.0F : -1.0F;  // as the estimator does (distance.h, finish_distances)
    }
    bool odd = !(bn > 0.0F) || !(berr > 0.0F) || !(bn < 1.0e18F) || !(berr < 1.0e18F);
    if (!is_l2) {
        odd = odd || !(fabsf(braw) >= 1e-5F) || !(fabsf(braw) < 1.0e18F);
    }
    float a_c = odd ? 0.0F : berr / (2.0F * bn);
    float b_c = odd ? 0.0F : (bn * bn - braw * braw) * a_c;
    odd = odd || !(a_c <= kRbMaxA) || !(fabsf(b_c) <= kRbMaxB) || !(bsum == static_cast<float>(bits));
    const bool holds = ids != nullptr ? ids[slot] != VSAG_AMD_INVALID_ID : slot < n;
    const uint32_t flags = (holds ? 1U : 0U) | (odd && holds ? 2U : 0U);
    f4const[slot] = make_float4(odd ? 0.0F : a_c, odd ? 0.0F : b_c, odd ? 0.0F : bsum, __uint_as_float(flags));
}

// f4group of tiles [first_tile, first_tile + ntiles); a thread per (tile, group).  Slots without a verdict (no code, or
// a code outside the pass) stay out; a group of nothing else gets a threshold nothing reaches (1e30 stays finite
// through the chain of multiply-adds it goes into).
__global__ void __launch_bounds__(256)
f4_group_kernel(const float4* f4const, uint64_t first_tile, uint64_t ntiles, float4* f4group) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= ntiles * 4) {
        return;
    }
    const uint64_t tile = first_tile + i / 4;
    const uint32_t group = static_cast<uint32_t>(i % 4), gi = group >> 1, gh = group & 1U;
    float lo_a = 1e30F, hi_a = -1e30F, lo_b = 1e30F, lo_s = 1e30F, hi_s = -1e30F;
    for (uint32_t c = 0; c < 16; ++c) {
        const float4 v = f4const[tile * kWave + 32 * gi + 8 * (c >> 2) + 4 * gh + (c & 3U)];
        if (__float_as_uint(v.w) == 1U) {
            lo_a = fminf(lo_a, v.x);
            hi_a = fmaxf(hi_a, v.x);
            lo_b = fminf(lo_b, v.y);
            lo_s = fminf(lo_s, v.z);
            hi_s = fmaxf(hi_s, v.z);
        }
    }
    // factor x constant is least at factor x centre - |factor| x half width
    f4group[(tile * 4 + group) * 2] = make_float4(0.5F * (lo_a + hi_a), 0.5F * (hi_a - lo_a), lo_b, 0.5F * (lo_s + hi_s));
    f4group[(tile * 4 + group) * 2 + 1] = make_float4(0.5F * (hi_s - lo_s), 0.0F, 0.0F, 0.0F);
}

// Renews f4tiles / f4const / f4group over tiles [first_tile, first_tile + ntiles) of a store of n codes.
static int
launch_f4(const vsag_amd_store* s, uint64_t n, uint64_t first_tile, uint64_t ntiles, hipStream_t st) {
    if (s->f4tiles == nullptr || ntiles == 0) {
        return 0;
    }
    hipLaunchKernelGGL(f4_from_tiles_kernel, dim3(static_cast<uint32_t>(div_up(ntiles * s->G * kWave, 256))), dim3(256), 0,
                       st, s->tiles, s->G, first_tile, ntiles, s->f4tiles);
    hipLaunchKernelGGL(f4_const_kernel, dim3(static_cast<uint32_t>(div_up(ntiles * kWave, 256))), dim3(256), 0, st, s->tiles,
                       s->G, s->meta, s->cap_tiles * kWave, s->metric == VSAG_AMD_METRIC_L2 ? 1 : 0,
                       s->nlist > 0 ? s->ids_dev : nullptr, n, first_tile * kWave, ntiles * kWave, s->f4const);
    hipLaunchKernelGGL(f4_group_kernel, dim3(static_cast<uint32_t>(div_up(ntiles * 4, 256))), dim3(256), 0, st, s->f4const,
                       first_tile, ntiles, s->f4group);
    VA_HIP(hipGetLastError());
    return 0;
}

static int
grow(vsag_amd_store* s, uint64_t need_tiles, hipStream_t st) {
    if (need_tiles <= s->cap_tiles) {
        return 0;
    }
    uint64_t cap = s->cap_tiles ? s->cap_tiles : 16;
    while (cap < need_tiles) {
        cap *= 2;
    }
    uint4* tiles = nullptr;
    uint32_t* meta = nullptr;
    size_t tile_bytes = cap * s->G * kWave * sizeof(uint4) + kTileSlackBytes;
    VA_HIP(hipMalloc(&tiles, tile_bytes));
    VA_HIP(hipMemsetAsync(tiles, 0, tile_bytes, st));
    if (s->nmeta > 0) {
        VA_HIP(hipMalloc(&meta, cap * kWave * s->nmeta * sizeof(uint32_t)));
        VA_HIP(hipMemsetAsync(meta, 0, cap * kWave * s->nmeta * sizeof(uint32_t), st));
    }
    if (s->ntiles > 0) {
        VA_HIP(hipMemcpyAsync(tiles, s->tiles, s->ntiles * s->G * kWave * sizeof(uint4), hipMemcpyDeviceToDevice, st));
        for (uint32_t m = 0; m < s->nmeta; ++m) {
            VA_HIP(hipMemcpyAsync(meta + m * cap * kWave, s->meta + m * s->cap_tiles * kWave,
                                  s->ntiles * kWave * sizeof(uint32_t), hipMemcpyDeviceToDevice, st));
        }
    }
    float* term = nullptr;
    if (s->pf_ymax != nullptr) {
        VA_HIP(hipMalloc(&term, cap * kWave * sizeof(float)));
        if (s->ntiles > 0) {
            VA_HIP(hipMemcpyAsync(term, s->pf_term, s->ntiles * kWave * sizeof(float), hipMemcpyDeviceToDevice, st));
        }
    }
    uint4* rows = nullptr;
    if (keeps_rows(s)) {
        s->row_granules = s->G + (s->nmeta > 0 ? 1 : 0);
        VA_HIP(hipMalloc(&rows, cap * kWave * s->row_granules * sizeof(uint4)));
        if (s->ntiles > 0) {
            VA_HIP(hipMemcpyAsync(rows, s->rows, s->ntiles * kWave * s->row_granules * sizeof(uint4),
                                  hipMemcpyDeviceToDevice, st));
        }
    }
    uint4* f4tiles = nullptr;
    float4* f4const = nullptr;
    float4* f4group = nullptr;
    if (keeps_f4(s)) {
        VA_HIP(hipMalloc(&f4tiles, cap * kWave * s->G * sizeof(uint4)));
        VA_HIP(hipMalloc(&f4const, cap * kWave * sizeof(float4)));
        VA_HIP(hipMalloc(&f4group, cap * 8 * sizeof(float4)));
        if (s->ntiles > 0) {
            VA_HIP(hipMemcpyAsync(f4tiles, s->f4tiles, s->ntiles * kWave * s->G * sizeof(uint4), hipMemcpyDeviceToDevice, st));
            VA_HIP(hipMemcpyAsync(f4const, s->f4const, s->ntiles * kWave * sizeof(float4), hipMemcpyDeviceToDevice, st));
            VA_HIP(hipMemcpyAsync(f4group, s->f4group, s->ntiles * 8 * sizeof(float4), hipMemcpyDeviceToDevice, st));
        }
    }
    VA_HIP(hipStreamSynchronize(st));
    for (void* p : {static_cast<void*>(s->f4tiles), static_cast<void*>(s->f4const), static_cast<void*>(s->f4group)}) {
        if (p != nullptr) {
            VA_HIP(hipFree(p));
        }
    }
    s->f4tiles = f4tiles;
    s->f4const = f4const;
    s->f4group = f4group;
    s->f4_slots = f4tiles != nullptr ? cap * kWave : 0;
    if (s->tiles) {
        VA_HIP(hipFree(s->tiles));
    }
    if (s->meta) {
        VA_HIP(hipFree(s->meta));
    }
    if (s->pf_term) {
        VA_HIP(hipFree(s->pf_term));
    }
    if (s->rows) {
        VA_HIP(hipFree(s->rows));
    }
    s->rows = rows;
    s->tiles = tiles;
    s->meta = meta;
    s->pf_term = term;
    s->cap_tiles = cap;
    return 0;
}

static RetileArgs
retile_args(const vsag_amd_store* s, const uint8_t* codes, uint64_t n) {
    RetileArgs a{};
    a.codes = codes;
    a.n = n;
    a.code_size = s->code_size;
    a.payload_bytes = s->payload_bytes;
    a.plane_bytes = s->plane_bytes;
    a.plane_granules = s->plane_granules;
    a.G = s->G;
    a.nmeta = s->nmeta;
    for (int m = 0; m < 4; ++m) {
        a.meta_offset[m] = s->meta_offset[m];
    }
    a.meta_is_u64 = s->meta_is_u64;
    a.tiles = s->tiles;
    a.meta = s->meta;
    a.meta_stride = s->cap_tiles * kWave;
    a.normalize = (s->kind == VSAG_AMD_KIND_FP32 && s->metric == VSAG_AMD_METRIC_COSINE && !s->stored_codes) ? 1 : 0;
    a.dim = s->dim;
    return a;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" uint64_t
vsag_amd_code_size(int kind, int metric, uint32_t dim, int rabitq_query_bits) {
    auto up = [](uint64_t v, uint64_t a) { return (v + a - 1) / a * a; };
    switch (kind) {
        case VSAG_AMD_KIND_FP32:
            return 4ull * dim;
        case VSAG_AMD_KIND_SQ8:
            return dim;
        case VSAG_AMD_KIND_SQ4:
            return (static_cast<uint64_t>(dim) * 4 + 7) / 8;
        case VSAG_AMD_KIND_SQ4_UNIFORM: {
            // sq4_uniform_quantizer.cpp:33-72: norm (u64) for l2 and cosine, two f32 sums for ip and cosine.
            bool norm = metric == VSAG_AMD_METRIC_L2 || metric == VSAG_AMD_METRIC_COSINE;
            bool sum = metric != VSAG_AMD_METRIC_L2;
            uint64_t align = norm ? 8 : 4;
            uint64_t size = up((dim + 1) / 2, align);
            if (norm) {
                size += up(8, align);
            }
            if (sum) {
                size += 2 * up(4, align);
            }
            return size;
        }
        case VSAG_AMD_KIND_SQ8_UNIFORM: {
            // sq8_uniform_quantizer.cpp:30-62: norm (u64) for l2, one f32 sum for ip and cosine.
            bool norm = metric == VSAG_AMD_METRIC_L2;
            uint64_t align = norm ? 8 : 4;
            return up(dim, align) + (norm ? 8 : 4);
        }
        case VSAG_AMD_KIND_RABITQ:
            return rabitq_code_size(dim, metric, (rabitq_query_bits & 255) ? rabitq_query_bits : (rabitq_query_bits | 4));
        case VSAG_AMD_KIND_PQFS:
            return (static_cast<uint64_t>(dim) + 1) / 2;  // dim = the number of subspaces here
        default:
            return 0;
    }
}

extern "C" int
vsag_amd_store_create(const vsag_amd_store_params_t* p, vsag_amd_store_t** out) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(p != nullptr && out != nullptr, "null params / output");
    *out = nullptr;
    VA_CHECK_ARG(p->kind >= VSAG_AMD_KIND_FP32 && p->kind <= VSAG_AMD_KIND_PQFS, "unknown store kind %d", p->kind);
    if (p->kind == VSAG_AMD_KIND_PQFS) {
        VA_CHECK_ARG(p->pq_dim >= 1 && p->dim % p->pq_dim == 0, "pq_dim(%u) does not divide evenly into dim(%u)", p->pq_dim,
                     p->dim);
        VA_CHECK_ARG(p->pq_dim <= kMaxPqDim, "pq_dim must be at most %u, got %u", kMaxPqDim, p->pq_dim);
        VA_CHECK_ARG(p->codebooks_dev != nullptr, "pqfs store needs codebooks_dev");
    }
    VA_CHECK_ARG(p->metric >= VSAG_AMD_METRIC_L2 && p->metric <= VSAG_AMD_METRIC_COSINE, "unknown metric %d",
                 p->metric);
    VA_CHECK_ARG(p->dim >= 1 && p->dim <= 65536, "dim must be in [1, 65536], got %u", p->dim);
    vsag_amd_store* s = new (std::nothrow) vsag_amd_store();
    if (s == nullptr) {
        return fail(VSAG_AMD_NO_ENOUGH_MEMORY, "host allocation failed");
    }
    s->kind = p->kind;
    s->metric = p->metric;
    s->dim = p->dim;
    s->query_bits = (p->rabitq_query_bits & 255) ? (p->rabitq_query_bits & 255) : 4;
    s->base_bits = (p->rabitq_query_bits >> 8) ? static_cast<uint32_t>(p->rabitq_query_bits >> 8) : 1U;
    if (p->kind == VSAG_AMD_KIND_RABITQ && s->base_bits != 1 && (s->query_bits != 32 || s->base_bits > 8)) {
        delete s;
        return fail(VSAG_AMD_INVALID_ARGUMENT, "multi-bit rabitq base codes take 2 to 8 bits and fp32 queries (got %u bits, "
                    "%d-bit queries)", s->base_bits, s->query_bits);
    }
    s->pq_dim = p->kind == VSAG_AMD_KIND_PQFS ? p->pq_dim : 0;
    s->code_size = static_cast<uint32_t>(
        vsag_amd_code_size(p->kind, p->metric, p->kind == VSAG_AMD_KIND_PQFS ? p->pq_dim : p->dim,
                           p->kind == VSAG_AMD_KIND_RABITQ ? rabitq_bits_word(s) : s->query_bits));
    uint32_t dims_per_granule = 16;
    auto up = [](uint64_t v, uint64_t a) { return (v + a - 1) / a * a; };
    int rc = 0;
    switch (p->kind) {
        case VSAG_AMD_KIND_FP32:
            s->payload_bytes = 4 * p->dim;
            dims_per_granule = 4;
            break;
        case VSAG_AMD_KIND_SQ8:
            s->payload_bytes = p->dim;
            dims_per_granule = 16;
            break;
        case VSAG_AMD_KIND_SQ4:
            s->payload_bytes = (p->dim + 1) / 2;
            dims_per_granule = 32;
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM: {
            s->payload_bytes = (p->dim + 1) / 2;
            dims_per_granule = 32;
            bool norm = p->metric == VSAG_AMD_METRIC_L2 || p->metric == VSAG_AMD_METRIC_COSINE;
            uint64_t align = norm ? 8 : 4;
            uint64_t off = up(s->payload_bytes, align);
            s->nmeta = 1;
            if (p->metric == VSAG_AMD_METRIC_L2) {
                s->meta_offset[0] = static_cast<uint32_t>(off);
                s->meta_is_u64 = 1;
            } else {
                s->meta_offset[0] = static_cast<uint32_t>(off + (norm ? up(8, align) : 0));
            }
            break;
        }
        case VSAG_AMD_KIND_SQ8_UNIFORM: {
            s->payload_bytes = p->dim;
            dims_per_granule = 16;
            uint64_t align = p->metric == VSAG_AMD_METRIC_L2 ? 8 : 4;
            s->nmeta = 1;
            s->meta_offset[0] = static_cast<uint32_t>(up(p->dim, align));
            s->meta_is_u64 = p->metric == VSAG_AMD_METRIC_L2 ? 1 : 0;
            s->nmeta = 2;
            s->meta_offset[1] = kMetaPayloadSum;
            break;
        }
        case VSAG_AMD_KIND_RABITQ: {
            s->planes = s->base_bits;
            s->plane_bytes = (p->dim + 7) / 8;
            s->payload_bytes = s->plane_bytes * s->planes;
            dims_per_granule = 128;
            uint32_t off = static_cast<uint32_t>(up(s->payload_bytes, 4));
            // (norm of the code,) norm, error, sum, raw norm (rabitq_quantizer.cpp:102-133); the code's norm exists for
            // multi-bit codes, the sum for query_bits != 32.  Word 2 holds whichever of those two the store has.
            s->nmeta = 4;
            if (s->base_bits != 1) {
                s->meta_offset[2] = off;
                off += 4;
            }
            s->meta_offset[0] = off;
            s->meta_offset[1] = off + 4;
            if (s->base_bits == 1) {
                s->meta_offset[2] = s->query_bits != 32 ? off + 8 : off + 4;
            }
            s->meta_offset[3] = p->metric != VSAG_AMD_METRIC_L2 ? s->code_size - 4 : off + 4;
            break;
        }
        case VSAG_AMD_KIND_PQFS:
            // a granule holds the 4-bit centroid indices of 32 subspaces (dpad counts subspaces for this kind)
            s->payload_bytes = s->code_size;
            dims_per_granule = 32;
            break;
    }
    if (s->plane_bytes == 0) {
        s->plane_bytes = s->payload_bytes;
    }
    s->plane_granules = static_cast<uint32_t>((s->plane_bytes + kGranule - 1) / kGranule);
    s->G = s->plane_granules * s->planes;
    s->dpad = s->plane_granules * dims_per_granule;

    auto fail_free = [&](int code) {
        vsag_amd_store_destroy(s);
        return code;
    };
    if (p->kind == VSAG_AMD_KIND_SQ8 || p->kind == VSAG_AMD_KIND_SQ4) {
        if (p->lower_bound_dev == nullptr || p->diff_dev == nullptr) {
            return fail_free(fail(VSAG_AMD_INVALID_ARGUMENT, "sq8/sq4 store needs lower_bound_dev and diff_dev"));
        }
        if (hipMalloc(&s->scale_dev, s->dpad * 4) != hipSuccess || hipMalloc(&s->lb_dev, s->dpad * 4) != hipSuccess ||
            hipMalloc(&s->diff_dev, s->dpad * 4) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_NO_ENOUGH_MEMORY, "hipMalloc of quantizer tables failed"));
        }
        float levels = p->kind == VSAG_AMD_KIND_SQ8 ? 255.0F : 15.0F;
        hipLaunchKernelGGL(scale_table_kernel, dim3((s->dpad + 255) / 256), dim3(256), 0, nullptr, p->lower_bound_dev,
                           p->diff_dev, p->dim, s->dpad, levels, s->scale_dev, s->lb_dev, s->diff_dev);
        if (hipStreamSynchronize(nullptr) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_INTERNAL_ERROR, "building the scale table failed"));
        }
    } else if (p->kind == VSAG_AMD_KIND_SQ4_UNIFORM || p->kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
        if (p->lower_bound_dev == nullptr) {
            return fail_free(fail(VSAG_AMD_INVALID_ARGUMENT, "uniform store needs lower_bound_dev = {lb, diff}"));
        }
        float b[2];
        if (hipMalloc(&s->bounds_dev, 8) != hipSuccess ||
            hipMemcpy(s->bounds_dev, p->lower_bound_dev, 8, hipMemcpyDeviceToDevice) != hipSuccess ||
            hipMemcpy(b, p->lower_bound_dev, 8, hipMemcpyDeviceToHost) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_INTERNAL_ERROR, "copying the uniform bounds failed"));
        }
        s->ulb = b[0];
        s->udiff = b[1];
        // sq4_uniform_quantizer.cpp:104 / sq8_uniform_quantizer.cpp:94: (diff / L) * (diff / L) in double.
        double levels = p->kind == VSAG_AMD_KIND_SQ4_UNIFORM ? 15.0 : 255.0;
        s->scalar_rate = static_cast<float>((s->udiff / levels) * (s->udiff / levels));
    } else if (p->kind == VSAG_AMD_KIND_RABITQ) {
        if (p->rotation_dev == nullptr || p->centroid_dev == nullptr) {
            return fail_free(fail(VSAG_AMD_INVALID_ARGUMENT, "rabitq store needs rotation_dev and centroid_dev"));
        }
        size_t rb = static_cast<size_t>(p->dim) * p->dim * 4;
        if (hipMalloc(&s->rotation_dev, rb) != hipSuccess || hipMalloc(&s->centroid_dev, p->dim * 4) != hipSuccess ||
            hipMemcpy(s->rotation_dev, p->rotation_dev, rb, hipMemcpyDeviceToDevice) != hipSuccess ||
            hipMemcpy(s->centroid_dev, p->centroid_dev, p->dim * 4, hipMemcpyDeviceToDevice) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_NO_ENOUGH_MEMORY, "copying the rabitq rotation failed"));
        }
    } else if (p->kind == VSAG_AMD_KIND_PQFS) {
        const size_t cb = static_cast<size_t>(p->dim) * 16 * 4;
        if (hipMalloc(&s->codebooks_dev, cb) != hipSuccess ||
            hipMemcpy(s->codebooks_dev, p->codebooks_dev, cb, hipMemcpyDeviceToDevice) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_NO_ENOUGH_MEMORY, "copying the pq codebooks failed"));
        }
    }
    // Stores the matrix cores can pre-select on keep a per-code term (and the largest norm, where a threshold needs it).
    if (p->kind == VSAG_AMD_KIND_FP32 || p->kind == VSAG_AMD_KIND_SQ8 || p->kind == VSAG_AMD_KIND_SQ4 ||
        ((p->kind == VSAG_AMD_KIND_SQ8_UNIFORM || p->kind == VSAG_AMD_KIND_SQ4_UNIFORM) && s->dpad <= 128)) {
        if (hipMalloc(&s->pf_ymax, 4) != hipSuccess || hipMemset(s->pf_ymax, 0, 4) != hipSuccess) {
            return fail_free(fail(VSAG_AMD_NO_ENOUGH_MEMORY, "hipMalloc of the norm scalar failed"));
        }
    }
    (void)rc;
    *out = s;
    return 0;
}

extern "C" int
vsag_amd_store_destroy(vsag_amd_store_t* s) {
    if (s == nullptr) {
        return 0;
    }
    void* ptrs[] = {s->scale_dev, s->lb_dev,  s->diff_dev, s->bounds_dev,    s->rotation_dev, s->centroid_dev,
                    s->tiles,     s->meta,    s->ids_dev,  s->list_tile_dev, s->pf_term,      s->pf_ymax,
                    s->rows,      s->slot_of_id_dev, s->residual_bias_dev, s->residual_centroids_dev,
                    s->list_sizes_dev, s->codebooks_dev, s->f4tiles, s->f4const, s->f4group};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    delete s;
    return 0;
}

extern "C" uint64_t
vsag_amd_store_size(const vsag_amd_store_t* s) {
    return s ? s->n : 0;
}

extern "C" int
vsag_amd_store_append(vsag_amd_store_t* s, const uint8_t* codes_dev, uint64_t n, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(s->nlist == 0, "append on a posting-list store");
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev != nullptr, "codes_dev is null");
    VA_CHECK_ARG(s->n + n < 0xFFFFFFFFull, "a store holds fewer than 2^32 - 1 codes");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint64_t need = div_up(s->n + n, kWave);
    VA_TRY(grow(s, need, st));
    RetileArgs a = retile_args(s, codes_dev, n);
    a.first_slot = s->n;
    uint64_t threads = n * s->G;
    hipLaunchKernelGGL(retile_kernel, dim3(static_cast<uint32_t>(div_up(threads, 256))), dim3(256), 0, st, a);
    VA_HIP(hipGetLastError());
    if (s->rows != nullptr) {
        hipLaunchKernelGGL(rows_from_tiles_kernel, dim3(static_cast<uint32_t>(div_up(n * s->row_granules, 256))), dim3(256),
                           0, st, s->tiles, s->G, s->row_granules, s->meta, s->cap_tiles * kWave, s->nmeta, s->n, n, s->rows);
        VA_HIP(hipGetLastError());
    }
    VA_TRY(launch_code_terms(s, s->n, n, st));
    VA_TRY(launch_f4(s, s->n + n, s->n / kWave, need - s->n / kWave, st));
    s->n += n;
    s->ntiles = need;
    return 0;
}

namespace {

// Frees the posting lists of a store (not its quantizer state).
int
drop_lists(vsag_amd_store* s) {
    for (void* p : {static_cast<void*>(s->tiles), static_cast<void*>(s->meta), static_cast<void*>(s->ids_dev),
                    static_cast<void*>(s->list_tile_dev), static_cast<void*>(s->slot_of_id_dev),
                    static_cast<void*>(s->residual_bias_dev), static_cast<void*>(s->list_sizes_dev)}) {
        if (p != nullptr) {
            VA_HIP(hipFree(p));
        }
    }
    if (s->pf_term_slots != 0 && s->pf_term != nullptr) {
        VA_HIP(hipFree(s->pf_term));
        s->pf_term = nullptr;
    }
    s->pf_term_slots = 0;
    for (void* p : {static_cast<void*>(s->f4tiles), static_cast<void*>(s->f4const), static_cast<void*>(s->f4group)}) {
        if (p != nullptr) {
            VA_HIP(hipFree(p));
        }
    }
    s->f4tiles = nullptr;
    s->f4const = nullptr;
    s->f4group = nullptr;
    s->f4_slots = 0;
    s->list_sizes_dev = nullptr;
    s->tiles = nullptr;
    s->meta = nullptr;
    s->ids_dev = nullptr;
    s->list_tile_dev = nullptr;
    s->slot_of_id_dev = nullptr;
    s->residual_bias_dev = nullptr;
    s->slot_of_id_cap = 0;
    s->cap_tiles = 0;
    s->ntiles = 0;
    s->n = 0;
    s->max_list_tiles = 0;
    s->list_sizes.clear();
    s->list_begin.clear();
    s->list_room.clear();
    return 0;
}

// Device buffers of one call that are freed whatever way the call ends.
struct Temporaries {
    std::vector<void*> ptrs;
    ~Temporaries() {
        for (void* p : ptrs) {
            if (p != nullptr) {
                (void)hipFree(p);
            }
        }
    }
    template <typename T>
    hipError_t
    alloc(T** out, size_t bytes) {
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, bytes ? bytes : 4);
        if (e == hipSuccess) {
            ptrs.push_back(p);
        }
        *out = static_cast<T*>(p);
        return e;
    }
};

// Appends n codes (reference byte layout, source row r gets inner id s->n + r) to the lists named by labels_dev, in
// input order inside every list.  bias_dev: per source row residual bias, or null.
int
append_to_lists(vsag_amd_store* s, const uint8_t* codes_dev, const int32_t* labels_dev, const float* bias_dev, uint64_t n,
                hipStream_t st) {
    const uint32_t nlist = s->nlist;
    if (n == 0) {
        return 0;
    }
    Temporaries tmp;
    // 1. how many new codes per list
    uint32_t* counts = nullptr;
    VA_HIP(tmp.alloc(&counts, (nlist + 1) * sizeof(uint32_t)));
    VA_HIP(hipMemsetAsync(counts, 0, (nlist + 1) * sizeof(uint32_t), st));
    hipLaunchKernelGGL(histogram_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, labels_dev, n,
                       nlist, counts, counts + nlist);
    std::vector<uint32_t> added(nlist + 1);
    VA_HIP(hipMemcpyAsync(added.data(), counts, (nlist + 1) * sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    VA_HIP(hipStreamSynchronize(st));
    VA_CHECK_ARG(added[nlist] == 0, "%u labels are outside [0, %u)", added[nlist], nlist);

    // 2. room: a list that outgrows its tiles moves every list to a new layout, with a quarter more room than it
    // needs now (the first fill takes exactly what it needs).
    const bool first_fill = s->n == 0;
    bool move = s->tiles == nullptr;
    std::vector<uint32_t> need(nlist), room(nlist);
    for (uint32_t l = 0; l < nlist; ++l) {
        need[l] = static_cast<uint32_t>(div_up(static_cast<uint64_t>(s->list_sizes[l]) + added[l], kWave));
        move = move || need[l] > s->list_room[l];
    }
    if (move) {
        uint64_t total = 0;
        std::vector<uint32_t> begin(nlist);
        for (uint32_t l = 0; l < nlist; ++l) {
            room[l] = need[l] > s->list_room[l] && !first_fill ? need[l] + need[l] / 4 + 1 : std::max(need[l], s->list_room[l]);
            begin[l] = static_cast<uint32_t>(total);
            total += room[l];
        }
        VA_CHECK_ARG(total * kWave < 0xFFFFFFFFull, "the posting lists would span 2^32 slots or more");
        const uint64_t cap = total > 0 ? total : 1;
        // Everything new is built beside the old; the store changes hands only when all of it exists.
        uint4* tiles = nullptr;
        uint32_t *meta = nullptr, *ids = nullptr, *lt = nullptr, *new_begin = nullptr;
        float* bias = nullptr;
        Temporaries fresh;
        VA_HIP(fresh.alloc(&tiles, cap * s->G * kWave * sizeof(uint4) + kTileSlackBytes));
        VA_HIP(hipMemsetAsync(tiles, 0, cap * s->G * kWave * sizeof(uint4), st));
        if (s->nmeta > 0) {
            VA_HIP(fresh.alloc(&meta, cap * kWave * s->nmeta * sizeof(uint32_t)));
            VA_HIP(hipMemsetAsync(meta, 0, cap * kWave * s->nmeta * sizeof(uint32_t), st));
        }
        VA_HIP(fresh.alloc(&ids, cap * kWave * sizeof(uint32_t)));
        hipLaunchKernelGGL(fill_u32_kernel, dim3(static_cast<uint32_t>(div_up(cap * kWave, 256))), dim3(256), 0, st, ids,
                           VSAG_AMD_INVALID_ID, cap * kWave);
        if (s->residual_centroids_dev != nullptr && s->metric == VSAG_AMD_METRIC_L2) {
            VA_HIP(fresh.alloc(&bias, cap * kWave * sizeof(float)));
            VA_HIP(hipMemsetAsync(bias, 0, cap * kWave * sizeof(float), st));
        }
        VA_HIP(fresh.alloc(&lt, 2 * static_cast<size_t>(nlist) * sizeof(uint32_t)));
        if (s->n > 0) {
            VA_HIP(tmp.alloc(&new_begin, nlist * sizeof(uint32_t)));
            VA_HIP(hipMemcpyAsync(new_begin, begin.data(), nlist * sizeof(uint32_t), hipMemcpyHostToDevice, st));
            RelocateArgs r{};
            r.old_tiles = s->tiles;
            r.new_tiles = tiles;
            r.G = s->G;
            r.old_lt = s->list_tile_dev;
            r.new_begin = new_begin;
            r.nlist = nlist;
            r.old_meta = s->meta;
            r.new_meta = meta;
            r.nmeta = s->nmeta;
            r.old_stride = s->cap_tiles * kWave;
            r.new_stride = cap * kWave;
            r.old_ids = s->ids_dev;
            r.new_ids = ids;
            r.slot_of_id = s->slot_of_id_dev;
            r.old_bias = s->residual_bias_dev;
            r.new_bias = bias;
            hipLaunchKernelGGL(relocate_tiles_kernel, dim3(static_cast<uint32_t>(s->cap_tiles)), dim3(256), 0, st, r);
            VA_HIP(hipGetLastError());
            VA_HIP(hipStreamSynchronize(st));
        }
        // The tile extents of the codes the lists hold now, at their new places: whatever fails from here on (the id map,
        // the temporaries and the sort below) leaves a store that a scan can still walk.
        std::vector<uint32_t> lt_now(2 * static_cast<size_t>(nlist));
        for (uint32_t l = 0; l < nlist; ++l) {
            lt_now[2 * l] = begin[l];
            lt_now[2 * l + 1] = begin[l] + static_cast<uint32_t>(div_up(static_cast<uint64_t>(s->list_sizes[l]), kWave));
        }
        VA_HIP(hipMemcpyAsync(lt, lt_now.data(), lt_now.size() * sizeof(uint32_t), hipMemcpyHostToDevice, st));
        VA_HIP(hipStreamSynchronize(st));
        for (void* p : {static_cast<void*>(s->tiles), static_cast<void*>(s->meta), static_cast<void*>(s->ids_dev),
                        static_cast<void*>(s->list_tile_dev), static_cast<void*>(s->residual_bias_dev)}) {
            if (p != nullptr) {
                (void)hipFree(p);
            }
        }
        fresh.ptrs.clear();  // the store owns them now
        s->tiles = tiles;
        s->meta = meta;
        s->ids_dev = ids;
        s->list_tile_dev = lt;
        s->residual_bias_dev = bias;
        s->cap_tiles = cap;
        s->list_begin = begin;
        s->list_room = room;
    }
    // 3. inner id -> slot map with room for the new ids
    if (s->n + n > s->slot_of_id_cap) {
        uint64_t cap = std::max<uint64_t>(s->n + n, s->slot_of_id_cap + s->slot_of_id_cap / 2);
        uint32_t* map = nullptr;
        VA_HIP(hipMalloc(&map, cap * sizeof(uint32_t)));
        if (s->n > 0) {
            VA_HIP(hipMemcpyAsync(map, s->slot_of_id_dev, s->n * sizeof(uint32_t), hipMemcpyDeviceToDevice, st));
            VA_HIP(hipStreamSynchronize(st));
        }
        if (s->slot_of_id_dev != nullptr) {
            (void)hipFree(s->slot_of_id_dev);
        }
        s->slot_of_id_dev = map;
        s->slot_of_id_cap = cap;
    }

    // 4. the new codes in list order (stable: the order the reference gets by appending vectors to their bucket one
    // after another, ivf.cpp:661-675 without a thread pool), each to the first free slots of its list
    std::vector<uint32_t> slot_base(nlist), lt_host(2 * static_cast<size_t>(nlist));
    uint32_t first_new = 0;
    for (uint32_t l = 0; l < nlist; ++l) {
        slot_base[l] = s->list_begin[l] * kWave + s->list_sizes[l] - first_new;  // modulo 2^32
        first_new += added[l];
    }
    int32_t* keys_out = nullptr;
    uint32_t *vals_in = nullptr, *vals_out = nullptr, *base_dev = nullptr, *dst_slot = nullptr;
    void* sort_tmp = nullptr;
    size_t sort_bytes = 0;
    VA_HIP(tmp.alloc(&keys_out, n * 4));
    VA_HIP(tmp.alloc(&vals_in, n * 4));
    VA_HIP(tmp.alloc(&vals_out, n * 4));
    VA_HIP(tmp.alloc(&dst_slot, n * 4));
    VA_HIP(tmp.alloc(&base_dev, nlist * 4));
    VA_HIP(hipMemcpyAsync(base_dev, slot_base.data(), nlist * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(iota_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, vals_in, n);
    int end_bit = 1;
    while ((1u << end_bit) < nlist) {
        ++end_bit;
    }
    VA_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, labels_dev, keys_out, vals_in, vals_out,
                                              static_cast<int>(n), 0, end_bit, st));
    VA_HIP(tmp.alloc(&sort_tmp, sort_bytes));
    VA_HIP(hipcub::DeviceRadixSort::SortPairs(sort_tmp, sort_bytes, labels_dev, keys_out, vals_in, vals_out,
                                              static_cast<int>(n), 0, end_bit, st));
    hipLaunchKernelGGL(list_slot_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, keys_out, n,
                       base_dev, dst_slot);
    RetileArgs a = retile_args(s, codes_dev, n);
    a.src_index = vals_out;
    a.dst_slot = dst_slot;
    a.ids = s->ids_dev;
    a.id_base = static_cast<uint32_t>(s->n);
    a.slot_of_id = s->slot_of_id_dev;
    a.bias_src = bias_dev;
    a.bias_dst = s->residual_bias_dev;
    hipLaunchKernelGGL(retile_kernel, dim3(static_cast<uint32_t>(div_up(n * s->G, 256))), dim3(256), 0, st, a);
    VA_HIP(hipGetLastError());

    // 5. the lists' new extents
    uint64_t used = 0;
    s->max_list_tiles = 0;
    for (uint32_t l = 0; l < nlist; ++l) {
        s->list_sizes[l] += added[l];
        lt_host[2 * l] = s->list_begin[l];
        lt_host[2 * l + 1] = s->list_begin[l] + need[l];
        used += need[l];
        s->max_list_tiles = std::max(s->max_list_tiles, need[l]);
    }
    VA_HIP(hipMemcpyAsync(s->list_tile_dev, lt_host.data(), lt_host.size() * sizeof(uint32_t), hipMemcpyHostToDevice, st));
    VA_HIP(hipMemcpyAsync(s->list_sizes_dev, s->list_sizes.data(), nlist * sizeof(uint32_t), hipMemcpyHostToDevice, st));
    VA_HIP(hipStreamSynchronize(st));
    s->ntiles = used;
    s->n += n;
    // The per-slot terms of the matrix-core passes over sq8 / sq4 lists (prefilter_i8.hip) and over fp32 and longer sq8
    // lists (prefilter.hip): recomputed over the whole buffer, which costs a pass over the codes (0.4 ms for ten million
    // sq8 codes) against the classification and encoding an append has behind it already.
    const bool list_terms = s->kind == VSAG_AMD_KIND_FP32 || s->kind == VSAG_AMD_KIND_SQ8 || s->kind == VSAG_AMD_KIND_SQ4;
    // (Residual lists: fp32 and sq8 under l2 / inner product go through the fp32 matrix cores, the int8 passes do not take
    // them.)
    const bool residual_ok = s->residual_centroids_dev == nullptr ||
                             ((s->kind == VSAG_AMD_KIND_FP32 || s->kind == VSAG_AMD_KIND_SQ8) &&
                              s->metric != VSAG_AMD_METRIC_COSINE);
    if (list_terms && s->pf_ymax != nullptr && residual_ok) {
        const uint64_t slots = s->cap_tiles * kWave;
        if (s->pf_term == nullptr || s->pf_term_slots < slots) {
            if (s->pf_term != nullptr) {
                VA_HIP(hipFree(s->pf_term));
                s->pf_term = nullptr;
            }
            VA_HIP(hipMalloc(&s->pf_term, slots * sizeof(float)));
            s->pf_term_slots = slots;
        }
        VA_TRY(launch_code_terms(s, 0, slots, st));
        VA_HIP(hipStreamSynchronize(st));
    }
    // The fp4 copy of 1-bit rabitq lists, renewed the same way.
    if (keeps_f4(s) && s->residual_centroids_dev == nullptr) {
        const uint64_t slots = s->cap_tiles * kWave;
        if (s->f4tiles == nullptr || s->f4_slots < slots) {
            for (void* p : {static_cast<void*>(s->f4tiles), static_cast<void*>(s->f4const), static_cast<void*>(s->f4group)}) {
                if (p != nullptr) {
                    VA_HIP(hipFree(p));
                }
            }
            s->f4tiles = nullptr;
            s->f4const = nullptr;
            s->f4group = nullptr;
            s->f4_slots = 0;
            VA_HIP(hipMalloc(&s->f4tiles, slots * s->G * sizeof(uint4)));
            VA_HIP(hipMalloc(&s->f4const, slots * sizeof(float4)));
            VA_HIP(hipMalloc(&s->f4group, s->cap_tiles * 8 * sizeof(float4)));
            s->f4_slots = slots;
        }
        VA_TRY(launch_f4(s, s->n, 0, s->cap_tiles, st));
        VA_HIP(hipStreamSynchronize(st));
    }
    return 0;
}

}  // namespace

extern "C" int
vsag_amd_store_set_lists(vsag_amd_store_t* s, const uint8_t* codes_dev, const int32_t* labels_dev, uint64_t n,
                         uint32_t nlist, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(nlist >= 1 && nlist <= (1u << 24), "nlist must be in [1, 2^24], got %u", nlist);
    VA_CHECK_ARG(n < 0xFFFFFFFFull, "a store holds fewer than 2^32 - 1 codes");
    VA_CHECK_ARG(n == 0 || (codes_dev && labels_dev), "null codes / labels");
    hipStream_t st = static_cast<hipStream_t>(stream);
    VA_HIP(hipStreamSynchronize(st));
    VA_TRY(drop_lists(s));
    s->nlist = nlist;
    s->list_sizes.assign(nlist, 0);
    s->list_begin.assign(nlist, 0);
    s->list_room.assign(nlist, 0);
    VA_HIP(hipMalloc(&s->list_sizes_dev, nlist * sizeof(uint32_t)));
    VA_HIP(hipMemsetAsync(s->list_sizes_dev, 0, nlist * sizeof(uint32_t), st));
    if (n == 0) {
        // Empty lists still need their offset table: every list begins and ends at tile 0.
        VA_HIP(hipMalloc(&s->list_tile_dev, 2 * static_cast<size_t>(nlist) * sizeof(uint32_t)));
        VA_HIP(hipMemsetAsync(s->list_tile_dev, 0, 2 * static_cast<size_t>(nlist) * sizeof(uint32_t), st));
        VA_HIP(hipMalloc(&s->tiles, kTileSlackBytes + kWave * s->G * sizeof(uint4)));
        VA_HIP(hipMalloc(&s->ids_dev, kWave * sizeof(uint32_t)));
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(256), 0, st, s->ids_dev, VSAG_AMD_INVALID_ID,
                           static_cast<uint64_t>(kWave));
        if (s->nmeta > 0) {
            VA_HIP(hipMalloc(&s->meta, kWave * s->nmeta * sizeof(uint32_t)));
        }
        s->cap_tiles = 1;
        VA_HIP(hipStreamSynchronize(st));
        return 0;
    }
    return append_to_lists(s, codes_dev, labels_dev, nullptr, n, st);
}

extern "C" int
vsag_amd_store_set_residual(vsag_amd_store_t* s, const float* centroids_dev, uint32_t nlist, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr && centroids_dev != nullptr, "null store / centroids");
    VA_CHECK_ARG(s->n == 0, "the residual centroids are set before the first code is stored");
    VA_CHECK_ARG(nlist >= 1 && (s->nlist == 0 || s->nlist == nlist), "nlist does not match the store's lists");
    if (s->residual_centroids_dev != nullptr) {
        VA_HIP(hipFree(s->residual_centroids_dev));
        s->residual_centroids_dev = nullptr;
    }
    const size_t bytes = static_cast<size_t>(nlist) * s->dim * sizeof(float);
    VA_HIP(hipMalloc(&s->residual_centroids_dev, bytes));
    VA_HIP(hipMemcpyAsync(s->residual_centroids_dev, centroids_dev, bytes, hipMemcpyDeviceToDevice,
                          static_cast<hipStream_t>(stream)));
    // The largest centroid norm bounds the per-slot bias of the residual arithmetic (2 |c| |y| + |c|^2), which the
    // matrix-core pass over residual lists needs for its error margin.
    std::vector<float> host(static_cast<size_t>(nlist) * s->dim);
    VA_HIP(hipMemcpyAsync(host.data(), centroids_dev, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    VA_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    double cmax = 0.0;
    for (uint32_t l = 0; l < nlist; ++l) {
        double sq = 0.0;
        for (uint32_t d = 0; d < s->dim; ++d) {
            const double v = host[static_cast<size_t>(l) * s->dim + d];
            sq += v * v;
        }
        cmax = std::max(cmax, std::sqrt(sq));
    }
    s->residual_cmax = std::isfinite(cmax) ? static_cast<float>(cmax * (1.0 + 1.0e-6)) : std::numeric_limits<float>::infinity();
    return 0;
}

extern "C" int
vsag_amd_store_append_lists(vsag_amd_store_t* s, const uint8_t* codes_dev, const int32_t* labels_dev,
                            const float* residual_bias_dev, uint64_t n, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(s->nlist > 0, "append_lists on a store without posting lists: call vsag_amd_store_set_lists first");
    VA_CHECK_ARG(s->n + n < 0xFFFFFFFFull, "a store holds fewer than 2^32 - 1 codes");
    VA_CHECK_ARG(n == 0 || (codes_dev && labels_dev), "null codes / labels");
    hipStream_t st = static_cast<hipStream_t>(stream);
    VA_HIP(hipStreamSynchronize(st));
    return append_to_lists(s, codes_dev, labels_dev, residual_bias_dev, n, st);
}

extern "C" int
vsag_amd_store_list_sizes(const vsag_amd_store_t* s, uint32_t* sizes, uint32_t nlist) {
    VA_CHECK_ARG(s != nullptr && sizes != nullptr, "null store / output");
    VA_CHECK_ARG(s->nlist == nlist, "store has %u lists, asked for %u", s->nlist, nlist);
    memcpy(sizes, s->list_sizes.data(), nlist * sizeof(uint32_t));
    return 0;
}

extern "C" int
vsag_amd_store_expect_stored_codes(vsag_amd_store_t* s, int on) {
    VA_CHECK_ARG(s != nullptr, "store is null");
    s->stored_codes = on != 0;
    return 0;
}
