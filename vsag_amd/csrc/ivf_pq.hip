// Posting lists of pqfs codes (PQ fast scan, at most 128 subspaces) against large query batches, on the int8
// matrix cores.
//
// A pqfs distance is a sum of table bytes, one per subspace: sum_i T_q[i][c_i], c_i the 4-bit centroid index of the
// code in subspace i and T_q the byte table of the query (pq_fastscan_quantizer.cpp:166-199, 299-361).  The reference
// forms it with byte shuffles over 32 codes at a time (PQFastScanLookUp32); a lane-per-code gather is bound by one
// memory instruction per (query, code, subspace).  Written as a contraction it is exact on v_mfma_i32_32x32x32_i8: the
// code side is the one-hot expansion of the indices (16 bytes per subspace, a single 1), the query side the table, and
// one matrix instruction covers two subspaces of 32 codes x 32 queries.  The table bytes are staged signed -- v - 128
// under inner product, 127 - v under l2, so that "distance <= bound" is "sum >= threshold" for both -- and the one-hot
// rows sum to one per subspace, so the shift is a per-query constant.  The map from the integer sum to the distance is
// monotone, so the test is an integer compare against a per-query threshold taken two units wide; what passes is
// recorded as (slot, sum) and turned into (distance, id) with the streaming kernel's own three operations, where the
// exact bound is applied (ivf_pq_finish_kernel).
//
// Work split (the grouping of ivf_i8.hip): a workgroup is a chunk of a list's tiles and up to 64 of the (query, list)
// pairs that probe the list.  The tables of its 64 queries stay in LDS for the whole kernel (16 bytes per subspace and
// query, 128 KB for 128 subspaces), laid out [subspace][query] so that the 32 lanes of an operand read 512 contiguous
// bytes.  Each of the eight waves walks its own tiles: it keeps a tile's code bytes in registers as they lie in the
// store (a lane per code), swaps the halves it needs with the lane 32 apart, builds the one-hot operands with a shift
// and four selects per subspace, and meets all 64 queries (four accumulators of 32 x 32).  Candidates of a pair go to
// one list per chunk through a counter in LDS; a list that overflows raises the query's gate and the streaming kernel
// rescans its lists.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);
int launch_ivf_clear_gated(uint32_t* gate, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t* partial_cnt,
                           const int32_t* buckets, uint32_t* gpairs, uint32_t gpairs_cap, uint32_t k, hipStream_t st);
uint32_t ivf_i8_lists_per_pair();

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kIvfPqPairs = 64;       // pairs per workgroup
constexpr uint32_t kIvfPqWaves = 8;        // two per SIMD: one waits for its table rows while the other multiplies
constexpr uint32_t kIvfPqMaxSubspaces = 128;
constexpr uint32_t kIvfPqChunkTiles = 32;  // as ivf_i8.hip: kIvfI8ChunkTiles, kIvfI8Chunks
constexpr uint32_t kIvfPqChunks = 4;

__host__ __device__ inline uint32_t
ivf_pq_list_chunks(uint32_t tiles) {
    const uint32_t chunks = (tiles + kIvfPqChunkTiles - 1) / kIvfPqChunkTiles;
    return chunks < kIvfPqChunks ? chunks : kIvfPqChunks;
}

// Per query the threshold of the staged sum (see the header): l2 acc = 127 pq_dim - sum, inner product
// acc = sum - 128 pq_dim; a pair passes when acc >= tq.  Two units wider than the bound asks for.
__global__ void __launch_bounds__(256)
ivf_pq_threshold_kernel(const uint32_t* bound, const float* qmeta, uint32_t qmeta_stride, int is_l2, uint32_t pq_dim,
                        uint64_t nq, int32_t* tq) {
    const uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q > nq) {
        return;
    }
    const int32_t never = 0x7FFFFFFF, always = static_cast<int32_t>(0x80000000U);
    if (q == nq) {
        tq[q] = never;  // the all-zero query row idle lanes point at
        return;
    }
    const uint32_t b = bound[q];
    const double diff = static_cast<double>(qmeta[q * qmeta_stride]);
    const double lower = static_cast<double>(qmeta[q * qmeta_stride + 1]);
    if (b == 0xFFFFFFFFU || !(diff > 0.0) || !(diff < 1.0e30) || !(fabs(lower) < 1.0e30)) {
        tq[q] = always;  // no bound, or a table without a range: everything passes and the exact check decides
        return;
    }
    const double bd = static_cast<double>(ordered_to_float(b));
    const double top = 255.0 * pq_dim + 2.0;
    if (is_l2) {
        // float(sum) / 255 * diff + lower <= bd  <=  sum <= (bd - lower) / diff * 255
        double x = (bd - lower) / diff * 255.0;
        x = floor(x + 1.0e-6 * fabs(x)) + 2.0;
        x = x > top ? top : (x < -2.0 ? -2.0 : x);
        tq[q] = 127 * static_cast<int32_t>(pq_dim) - static_cast<int32_t>(x);
    } else {
        // 1 - (float(sum) / 255 * diff + lower) <= bd  <=  sum >= (1 - bd - lower) / diff * 255
        double y = (1.0 - bd - lower) / diff * 255.0;
        y = floor(y - 1.0e-6 * fabs(y)) - 2.0;
        y = y > top ? top : (y < -2.0 ? -2.0 : y);
        tq[q] = static_cast<int32_t>(y) - 128 * static_cast<int32_t>(pq_dim);
    }
}

struct IvfPqArgs {
    const uint4* tiles;
    uint32_t G;                  // granules per code (<= 4)
    uint32_t pq_dim;
    const uint32_t* list_tile;   // 2 nlist: first tile and end of the used tiles of every list
    const uint32_t* pair_off;    // nlist + 1
    const uint32_t* item_off;    // nlist + 1: workgroups per list (64 pairs x tile chunks), prefix sums
    const uint32_t* sorted_pair; // pair index (q * nprobe + p) grouped by list
    uint32_t nlist, nprobe;
    uint32_t dummy_query;        // index of the all-zero query row
    const uint32_t* qtab;        // byte tables, 16 bytes per subspace
    uint32_t qstride;            // words per query
    const int32_t* tq;           // per query (+ the dummy row)
    uint32_t k;                  // capacity of a list
    uint32_t lists_per_pair;
    uint64_t* partial;           // [pair][lists_per_pair][k] records
    uint32_t* partial_cnt;
    uint32_t* gate;              // per query: raised when one of its lists overflowed; gate[nq] counts them
};

// The one-hot operand of a subspace: 16 bytes, byte `nib` is 1.
__device__ inline intx4
pq_one_hot(uint32_t nib) {
    const uint32_t one = 1U << ((nib & 3U) * 8U);
    const uint32_t sel = nib >> 2;
    return intx4{static_cast<int>(sel == 0 ? one : 0U), static_cast<int>(sel == 1 ? one : 0U),
                 static_cast<int>(sel == 2 ? one : 0U), static_cast<int>(sel == 3 ? one : 0U)};
}

template <int METRIC>
__global__ void __launch_bounds__(kIvfPqWaves * kWave)
ivf_pq_kernel(IvfPqArgs p) {
    extern __shared__ uint4 lut[];  // [subspace][kIvfPqPairs]
    __shared__ uint32_t cnt[kIvfPqPairs];
    __shared__ uint32_t spair[kIvfPqPairs];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint32_t item = blockIdx.x;
    cu32_p ioff = as_const(p.item_off);
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
    // Items of a list: (block of 64 pairs) x (tile chunk), chunk fastest.
    const uint32_t list_begin = as_const(p.list_tile)[2 * b], list_end = as_const(p.list_tile)[2 * b + 1];
    const uint32_t chunks = ivf_pq_list_chunks(list_end - list_begin);
    if (chunks == 0) {
        return;
    }
    const uint32_t per = (list_end - list_begin + chunks - 1) / chunks;
    const uint32_t chunk = (item - ioff[b]) % chunks;
    const uint32_t group = (item - ioff[b]) / chunks;
    uint32_t tile_begin = list_begin + chunk * per;
    tile_begin = tile_begin < list_end ? tile_begin : list_end;
    const uint32_t tile_end = tile_begin + per < list_end ? tile_begin + per : list_end;
    if (tile_begin >= tile_end) {
        return;  // an empty chunk: its lists keep their zero counts
    }
    const uint32_t pbeg = as_const(p.pair_off)[b] + group * kIvfPqPairs;
    const uint32_t pend = as_const(p.pair_off)[b + 1];
    // Matrix steps, two subspaces each: whole granules (a granule's 16 bytes are 16 steps), so that the loop over a
    // granule has no branch in it; the tables are zero behind the last subspace and so are the codes' indices.
    const uint32_t nsteps = 16 * p.G;

    // The tables of the workgroup's queries into LDS, staged signed; zero behind the last subspace.
    {
        const uint32_t qi = tid & (kIvfPqPairs - 1);
        const uint32_t idx = pbeg + qi;
        const bool live = idx < pend;
        const uint32_t pr = live ? as_const(p.sorted_pair)[idx] : 0xFFFFFFFFU;
        const uint32_t q = live ? pr / p.nprobe : p.dummy_query;
        if (tid < kIvfPqPairs) {
            cnt[tid] = 0;
            spair[tid] = pr;
        }
        const uint4* row = reinterpret_cast<const uint4*>(p.qtab + static_cast<uint64_t>(q) * p.qstride);
        const uint32_t flip = METRIC == VSAG_AMD_METRIC_L2 ? 0x7F7F7F7FU : 0x80808080U;
        for (uint32_t sub = tid / kIvfPqPairs; sub < 2 * nsteps; sub += kIvfPqWaves * kWave / kIvfPqPairs) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (sub < p.pq_dim) {
                v = row[sub];
                v = make_uint4(v.x ^ flip, v.y ^ flip, v.z ^ flip, v.w ^ flip);
            }
            lut[sub * kIvfPqPairs + qi] = v;
        }
    }
    __syncthreads();

    int32_t tq[2];
    uint32_t pair[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        pair[j] = spair[32 * j + l32];
        tq[j] = p.tq[pair[j] != 0xFFFFFFFFU ? pair[j] / p.nprobe : p.dummy_query];
    }

    // A wave's tiles: tile_begin + wave, + 8, ...; the code bytes of the next tile are fetched while this one is met.
    uint4 cw[4], nw[4];
    auto fetch = [&](uint32_t tile, uint4(&regs)[4]) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            regs[g] = make_uint4(0, 0, 0, 0);
            if (tile < tile_end && static_cast<uint32_t>(g) < p.G) {
                regs[g] = p.tiles[(static_cast<uint64_t>(tile) * p.G + g) * kWave + lane];
            }
        }
    };
    fetch(tile_begin + wave, cw);
    for (uint32_t tile = tile_begin + wave; tile < tile_end; tile += kIvfPqWaves) {
        fetch(tile + kIvfPqWaves, nw);
        intx16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0;
                }
            }
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (static_cast<uint32_t>(g) >= p.G) {
                break;
            }
            const uint32_t w4[4] = {cw[g].x, cw[g].y, cw[g].z, cw[g].w};
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                // Byte s of a code holds subspaces 2 s (low nibble) and 2 s + 1 (high nibble).  In a matrix step the
                // lanes below 32 supply subspace 2 s of codes lane and lane + 32, the lanes from 32 on subspace
                // 2 s + 1 of codes lane - 32 and lane: each takes what it lacks from the lane 32 apart.
                const uint32_t own = w4[m];
                const uint32_t oth = __shfl_xor(own, 32);
                const uint32_t n0 = (half ? (oth >> 4) : own) & 0x0F0F0F0FU;  // codes 0 .. 31 of the tile
                const uint32_t n1 = (half ? (own >> 4) : oth) & 0x0F0F0F0FU;  // codes 32 .. 63
#pragma unroll
                for (int bb = 0; bb < 4; ++bb) {
                    const uint32_t s = 16U * g + 4U * m + bb;
                    const intx4 a0 = pq_one_hot((n0 >> (8 * bb)) & 15U);
                    const intx4 a1 = pq_one_hot((n1 >> (8 * bb)) & 15U);
                    const uint4 t0 = lut[(2 * s + half) * kIvfPqPairs + l32];
                    const uint4 t1 = lut[(2 * s + half) * kIvfPqPairs + 32 + l32];
                    const intx4 b0 = intx4{static_cast<int>(t0.x), static_cast<int>(t0.y), static_cast<int>(t0.z),
                                           static_cast<int>(t0.w)};
                    const intx4 b1 = intx4{static_cast<int>(t1.x), static_cast<int>(t1.y), static_cast<int>(t1.z),
                                           static_cast<int>(t1.w)};
                    acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, acc[0][0], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b0, acc[1][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b1, acc[0][1], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, acc[1][1], 0, 0, 0);
                }
            }
        }
        // Verdicts.  Element e of a lane is code 32 i + 8 (e / 4) + 4 (lane / 32) + e % 4 of the tile against query
        // 32 j + lane % 32.  Nearly nothing passes: a max over the sixteen elements and one compare per block.
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                int32_t best = acc[i][j][0];
#pragma unroll
                for (int e = 1; e < 16; ++e) {
                    best = max(best, acc[i][j][e]);
                }
                if (__ballot(best >= tq[j]) == 0) {
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    if (acc[i][j][e] >= tq[j] && pair[j] != 0xFFFFFFFFU) {
                        const uint64_t slot = static_cast<uint64_t>(tile) * kWave + 32 * i + 8 * (e >> 2) + 4 * half + (e & 3);
                        const uint32_t pos = atomicAdd(&cnt[32 * j + l32], 1U);
                        if (pos < p.k) {
                            const uint64_t list = static_cast<uint64_t>(pair[j]) * p.lists_per_pair + chunk;
                            p.partial[list * p.k + pos] = (slot << 32) | static_cast<uint32_t>(acc[i][j][e]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            cw[g] = nw[g];
        }
    }
    __syncthreads();
    if (tid < kIvfPqPairs) {
        const uint32_t pr = spair[tid];
        if (pr != 0xFFFFFFFFU) {
            const uint32_t n = cnt[tid];
            // k + 1 for a list that overflowed: that is how the pair is told from the query's other pairs afterwards
            p.partial_cnt[static_cast<uint64_t>(pr) * p.lists_per_pair + chunk] = n <= p.k ? n : p.k + 1;
            if (n > p.k) {
                const uint32_t q = pr / p.nprobe;
                if (atomicExch(&p.gate[q], 1U) == 0U) {
                    atomicAdd(&p.gate[p.dummy_query], 1U);
                }
            }
        }
    }
}

// One thread per list: its (slot, staged sum) records become (distance, id) keys through the streaming kernel's own
// operations on the same integer; records of empty slots and of distances beyond the query's bound are dropped.
struct IvfPqFinishArgs {
    uint64_t* partial;
    uint32_t* partial_cnt;
    uint64_t lists;  // pairs x lists per pair
    uint32_t k, nprobe, p0, per_pair;
    const uint32_t* ids;
    uint32_t pq_dim;
    const float* qmeta;
    uint32_t qmeta_stride;
    const uint32_t* bound;
};

template <int METRIC>
__global__ void __launch_bounds__(256)
ivf_pq_finish_kernel(IvfPqFinishArgs p) {
    const uint64_t list = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (list >= p.lists) {
        return;
    }
    const uint64_t pair = list / p.per_pair;
    if (pair % p.nprobe < p.p0) {
        return;
    }
    const uint32_t count = p.partial_cnt[list];
    if (count == 0) {
        return;
    }
    const uint64_t q = pair / p.nprobe;
    const float diff = p.qmeta[q * p.qmeta_stride], lower = p.qmeta[q * p.qmeta_stride + 1];
    const uint32_t bound = p.bound[q];
    uint64_t* keys = p.partial + list * p.k;
    uint32_t kept = 0;
    for (uint32_t i = 0; i < count; ++i) {
        const uint64_t rec = keys[i];
        const uint64_t slot = rec >> 32;
        const int32_t acc = static_cast<int32_t>(static_cast<uint32_t>(rec));
        const uint32_t id = p.ids[slot];
        if (id == VSAG_AMD_INVALID_ID) {
            continue;
        }
        const int32_t sum = METRIC == VSAG_AMD_METRIC_L2 ? 127 * static_cast<int32_t>(p.pq_dim) - acc
                                                         : acc + 128 * static_cast<int32_t>(p.pq_dim);
        const float v = static_cast<float>(sum) / 255.0F * diff + lower;
        const float dist = METRIC == VSAG_AMD_METRIC_L2 ? v : 1.0F - v;
        if (float_to_ordered(dist) <= bound) {
            keys[kept++] = make_key(dist, id);
        }
    }
    p.partial_cnt[list] = kept;
}

bool
ivf_pq_supports(const vsag_amd_store* s) {
    return s->kind == VSAG_AMD_KIND_PQFS && s->nlist > 0 && s->pq_dim <= kIvfPqMaxSubspaces && s->G <= 4;
}

uint32_t
ivf_pq_pairs_per_item() {
    return kIvfPqPairs;
}

// The pairs of probe columns [p0, nprobe) are grouped by list (pair_off, sorted_pair) and item_off counts workgroups
// per list (blocks of 64 pairs x tile chunks: offsets_kernel with T = 64, kIvfPqChunkTiles, kIvfPqChunks); `bound`
// holds what the first columns left.  tq: nq + 1 words; gate: nq + 2 words, zeroed.
int
launch_ivf_pq(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
              const uint32_t* pair_off, const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound,
              int32_t* tq, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const int32_t* buckets,
              uint32_t* gpairs, uint32_t gpairs_cap, hipStream_t st) {
    const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
    hipLaunchKernelGGL(ivf_pq_threshold_kernel, dim3(static_cast<uint32_t>(div_up(nq + 1, 256))), dim3(256), 0, st, bound,
                       a.qmeta, a.qmeta_stride, l2 ? 1 : 0, s->pq_dim, nq, tq);
    IvfPqArgs p{};
    p.tiles = s->tiles;
    p.G = s->G;
    p.pq_dim = s->pq_dim;
    p.list_tile = s->list_tile_dev;
    p.pair_off = pair_off;
    p.item_off = item_off;
    p.sorted_pair = sorted_pair;
    p.nlist = s->nlist;
    p.nprobe = nprobe;
    p.dummy_query = static_cast<uint32_t>(nq);
    p.qtab = a.qtab;
    p.qstride = a.qstride;
    p.tq = tq;
    p.k = kcand;
    p.lists_per_pair = ivf_i8_lists_per_pair();
    p.partial = partial;
    p.partial_cnt = partial_cnt;
    p.gate = gate;
    const size_t lds = static_cast<size_t>(32) * s->G * kIvfPqPairs * sizeof(uint4);
    static bool attr_set = false;
    if (!attr_set) {
        const int bytes = static_cast<int>(kIvfPqMaxSubspaces * kIvfPqPairs * sizeof(uint4));
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ivf_pq_kernel<VSAG_AMD_METRIC_L2>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        VA_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ivf_pq_kernel<VSAG_AMD_METRIC_IP>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        attr_set = true;
    }
    // At most one partly filled block of pairs per probed list, each cut into at most kIvfPqChunks items.
    const uint64_t pairs = nq * (nprobe - p0);
    const uint64_t max_items =
        (div_up(pairs, static_cast<uint64_t>(kIvfPqPairs)) + std::min<uint64_t>(s->nlist, pairs)) * kIvfPqChunks;
    const dim3 grid(static_cast<uint32_t>(max_items));
    timing_begin(st);
    if (l2) {
        hipLaunchKernelGGL(ivf_pq_kernel<VSAG_AMD_METRIC_L2>, grid, dim3(kIvfPqWaves * kWave), lds, st, p);
    } else {
        hipLaunchKernelGGL(ivf_pq_kernel<VSAG_AMD_METRIC_IP>, grid, dim3(kIvfPqWaves * kWave), lds, st, p);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    VA_TRY(launch_ivf_clear_gated(gate, nq, nprobe, p0, partial_cnt, buckets, gpairs, gpairs_cap, kcand, st));
    IvfPqFinishArgs f{};
    f.partial = partial;
    f.partial_cnt = partial_cnt;
    f.per_pair = p.lists_per_pair;
    f.lists = nq * nprobe * f.per_pair;
    f.k = kcand;
    f.nprobe = nprobe;
    f.p0 = p0;
    f.ids = s->ids_dev;
    f.pq_dim = s->pq_dim;
    f.qmeta = a.qmeta;
    f.qmeta_stride = a.qmeta_stride;
    f.bound = bound;
    const dim3 fgrid(static_cast<uint32_t>(div_up(f.lists, 256)));
    if (l2) {
        hipLaunchKernelGGL(ivf_pq_finish_kernel<VSAG_AMD_METRIC_L2>, fgrid, dim3(256), 0, st, f);
    } else {
        hipLaunchKernelGGL(ivf_pq_finish_kernel<VSAG_AMD_METRIC_IP>, fgrid, dim3(256), 0, st, f);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
