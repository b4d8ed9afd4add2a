// Codes out of a store in the reference's byte layout: what FlattenDataCell::Serialize (src/datacell/
// flatten_datacell.h:481-486, io/common/basic_io.h:196-207) and BucketDataCell::Serialize (src/datacell/
// bucket_datacell.h:892-904) write.  The store keeps a code as 16-byte granules in tiles plus 4-byte metadata words;
// this is the inverse of retile_kernel (store.hip).
#include "store.h"

namespace vsag_amd {

struct UntileArgs {
    const uint4* tiles;
    uint32_t G;
    const uint32_t* meta;
    uint64_t meta_stride;
    uint32_t nmeta;
    uint32_t meta_offset[4];
    uint32_t meta_is_u64;
    uint32_t code_size, payload_bytes;
    uint32_t plane_bytes, plane_granules;  // the payload as zero-padded planes (see vsag_amd_store)
    int nibbles;               // the u64 word is the sum of squared 4-bit values (sq4_uniform), else of squared bytes
    uint64_t n;
    uint64_t first_slot;       // slot of output row i: first_slot + i ...
    const uint32_t* src_slot;  // ... or src_slot[i]
    uint8_t* out;              // n x code_size
};

// One thread per (code, granule).
__global__ void __launch_bounds__(256)
untile_kernel(UntileArgs a) {
    const uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint64_t i = gid / a.G;
    const uint32_t j = static_cast<uint32_t>(gid % a.G);
    if (i >= a.n) {
        return;
    }
    const uint64_t slot = a.src_slot != nullptr ? a.src_slot[i] : a.first_slot + i;
    const uint64_t tile = slot / kWave;
    const uint32_t lane = static_cast<uint32_t>(slot % kWave);
    uint8_t* dst = a.out + i * a.code_size;
    const uint4 v = a.tiles[(tile * a.G + j) * kWave + lane];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const uint32_t plane = j / a.plane_granules;
    for (uint32_t b = 0; b < 16; ++b) {
        const uint32_t off = 16 * (j - plane * a.plane_granules) + b;
        if (off < a.plane_bytes) {
            dst[plane * a.plane_bytes + off] = static_cast<uint8_t>(w[b >> 2] >> (8 * (b & 3)));
        }
    }
    if (j != 0) {
        return;
    }
    // Behind the payload: alignment bytes (zero) and the metadata words.
    for (uint32_t off = a.payload_bytes; off < a.code_size; ++off) {
        dst[off] = 0;
    }
    for (uint32_t m = 0; m < a.nmeta; ++m) {
        if (a.meta_offset[m] == kMetaPayloadSum) {
            continue;  // no field of the code
        }
        uint8_t* p = dst + a.meta_offset[m];
        if ((a.meta_is_u64 >> m) & 1U) {
            // The store keeps this integer as a float; the code holds it exactly: the sum of the squared code values
            // (sq8_uniform_quantizer.cpp:121-127, sq4_uniform_quantizer.cpp:134-147).
            uint64_t sum = 0;
            for (uint32_t g = 0; g < a.G; ++g) {
                const uint4 c = a.tiles[(tile * a.G + g) * kWave + lane];
                const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
                for (uint32_t b = 0; b < 16; ++b) {
                    if (16 * g + b < a.payload_bytes) {
                        const uint32_t byte = (cw[b >> 2] >> (8 * (b & 3))) & 255U;
                        if (a.nibbles) {
                            sum += (byte & 15U) * (byte & 15U) + (byte >> 4) * (byte >> 4);
                        } else {
                            sum += byte * byte;
                        }
                    }
                }
            }
            for (int b = 0; b < 8; ++b) {
                p[b] = static_cast<uint8_t>(sum >> (8 * b));
            }
        } else {
            const uint32_t word = a.meta[m * a.meta_stride + slot];
            for (int b = 0; b < 4; ++b) {
                p[b] = static_cast<uint8_t>(word >> (8 * b));
            }
        }
    }
}

// Output row i of a list-by-list export: list l = the last one with offsets[l] <= i, position i - offsets[l].
__global__ void __launch_bounds__(256)
list_rows_kernel(const uint32_t* offsets, uint32_t nlist, const uint32_t* list_tile, const uint32_t* ids,
                 const float* bias, uint64_t n, uint32_t* slots, uint32_t* ids_out, float* bias_out) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    uint32_t lo = 0, hi = nlist;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (offsets[mid] <= i) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const uint32_t slot = list_tile[2 * lo] * kWave + static_cast<uint32_t>(i - offsets[lo]);
    slots[i] = slot;
    ids_out[i] = ids[slot];
    if (bias_out != nullptr) {
        bias_out[i] = bias != nullptr ? bias[slot] : 0.0F;
    }
}

static UntileArgs
untile_args(const vsag_amd_store* s, uint64_t n, uint8_t* out) {
    UntileArgs a{};
    a.tiles = s->tiles;
    a.G = s->G;
    a.meta = s->meta;
    a.meta_stride = s->cap_tiles * kWave;
    a.nmeta = s->nmeta;
    for (int m = 0; m < 4; ++m) {
        a.meta_offset[m] = s->meta_offset[m];
    }
    a.meta_is_u64 = s->meta_is_u64;
    a.code_size = s->code_size;
    a.payload_bytes = s->payload_bytes;
    a.plane_bytes = s->plane_bytes;
    a.plane_granules = s->plane_granules;
    a.nibbles = s->kind == VSAG_AMD_KIND_SQ4_UNIFORM ? 1 : 0;
    a.n = n;
    a.out = out;
    return a;
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" int
vsag_amd_store_export_codes(const vsag_amd_store_t* s, uint64_t first, uint64_t n, uint8_t* codes_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(s->nlist == 0, "a posting-list store is exported list by list");
    VA_CHECK_ARG(first <= s->n && n <= s->n - first, "codes [%llu, %llu) are not in the store",
                 static_cast<unsigned long long>(first), static_cast<unsigned long long>(first + n));
    if (n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev != nullptr, "null output");
    UntileArgs a = untile_args(s, n, codes_dev);
    a.first_slot = first;
    hipLaunchKernelGGL(untile_kernel, dim3(static_cast<uint32_t>(div_up(n * s->G, 256))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_store_export_lists(const vsag_amd_store_t* s, uint8_t* codes_dev, uint32_t* ids_dev, float* bias_dev,
                            void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr && s->nlist > 0, "not a posting-list store");
    if (s->n == 0) {
        return 0;
    }
    VA_CHECK_ARG(codes_dev != nullptr && ids_dev != nullptr, "null output");
    hipStream_t st = static_cast<hipStream_t>(stream);
    std::vector<uint32_t> offsets(s->nlist + 1, 0);
    for (uint32_t l = 0; l < s->nlist; ++l) {
        offsets[l + 1] = offsets[l] + s->list_sizes[l];
    }
    VA_CHECK_ARG(offsets[s->nlist] == s->n, "list sizes do not add up to the store size");
    uint32_t* offsets_dev = nullptr;
    uint32_t* slots_dev = nullptr;
    VA_HIP(hipMalloc(reinterpret_cast<void**>(&offsets_dev), offsets.size() * sizeof(uint32_t)));
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&slots_dev), s->n * sizeof(uint32_t));
    if (e == hipSuccess) {
        e = hipMemcpyAsync(offsets_dev, offsets.data(), offsets.size() * sizeof(uint32_t), hipMemcpyHostToDevice, st);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(list_rows_kernel, dim3(static_cast<uint32_t>(div_up(s->n, 256))), dim3(256), 0, st, offsets_dev,
                           s->nlist, s->list_tile_dev, s->ids_dev, s->residual_bias_dev, s->n, slots_dev, ids_dev,
                           bias_dev);
        UntileArgs a = untile_args(s, s->n, codes_dev);
        a.src_slot = slots_dev;
        hipLaunchKernelGGL(untile_kernel, dim3(static_cast<uint32_t>(div_up(s->n * s->G, 256))), dim3(256), 0, st, a);
        e = hipGetLastError();
    }
    if (e == hipSuccess) {
        e = hipStreamSynchronize(st);  // the host vector and the temporaries go away
    }
    (void)hipFree(offsets_dev);
    (void)hipFree(slots_dev);
    VA_HIP(e);
    return 0;
}
