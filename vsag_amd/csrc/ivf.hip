// Batched IVF search: exact routing, posting-list scan with a fused per-(query, list) top-k, per-query
// merge, fp32 rerank (IVF::search<KNN_SEARCH>, src/algorithm/ivf/ivf.cpp:1693-1828; BucketDataCell::
// ScanBucketById, src/datacell/bucket_datacell.h:527-572; FlatBucketSearcher::Search,
// src/algorithm/ivf/flat_bucket_searcher.cpp:26-138; FlattenReorder::Reorder,
// src/impl/reorder/flatten_reorder.cpp:52-114).
//
// The reference walks "for each query, for each probed list".  Here the (query, list) pairs of the whole
// batch are regrouped by list on the device, so that one wave streams a posting list once for up to T
// queries that probe it.  A pair keeps its own LDS selector; what it cannot beat is cut off early by a
// per-query bound shared through global memory: the first probed list of every query is scanned in a
// first launch and its kcand-th distance seeds the bound for the remaining lists.  The bound only ever
// drops candidates that cannot be in the final kcand, so the result does not depend on scheduling.
//
// Few queries make few (query, list) pairs, and a wave per pair would leave the machine idle while each
// wave walks a whole list.  Then lists are cut into chunks of a few tiles, a work item is (list, query
// group, chunk), all probe columns go in one launch, and the cold waves learn a bound from each other's
// first tiles as in the flat scan.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

struct ScanPlanIvf {
    int T;
    uint32_t S;
    QueryLayout ql;
    size_t qcode_bytes;
    uint64_t npairs;
    uint32_t tiles_per_item;  // 0xFFFFFFFF: a work item walks its whole list
    uint32_t chunks_max;      // partial lists per (query, list) pair
    bool chunked;             // one launch over all probe columns, seeded cold start
    bool seeded;
    bool mfma;                // probe columns behind the first go through the int8 matrix cores (ivf_i8.hip)
    bool planes;              // ... with sq8 codes: two int8 planes per query, records rescored (prefilter_i8.hip)
    bool bits1;               // ... with rabitq codes: expanded bits, records rescored (prefilter_rb.hip)
    bool pq;                  // ... with pqfs codes: one-hot centroid indices against the byte tables (ivf_pq.hip)
    bool h16;                 // ... sq8 codes beyond 128 dimensions: the fp16 matrix cores, records rescored
    bool f32;                 // ... with fp32 codes (sq8 beyond 128 dimensions): the fp32 matrix cores, records rescored
                              // (prefilter.hip)
};

uint64_t rabitq_query_code_size(uint32_t dim, int metric, int query_bits);
int scan_contraction_mode(const vsag_amd_store* s);
void note_last_scan(int query_tile, uint64_t passes, uint64_t bytes_per_pass);
bool ivf_i8_supports(const vsag_amd_store* s);
uint32_t ivf_i8_lists_per_pair();
// sq8 lists: the two-plane test of prefilter_i8.hip over the same work split, records rescored by prefilter.hip.
bool ivf_sq8_i8_supports(const vsag_amd_store* s);
size_t ivf_sq8_i8_query_bytes(uint64_t nq);
size_t ivf_sq8_i8_scalar_floats(uint64_t nq);
size_t ivf_sq8_i8_tau_words(uint64_t nq);
uint32_t ivf_rescore_capacity();
int launch_ivf_sq8_i8(const vsag_amd_store* s, const float* qtab, uint32_t qstride, const float* qmeta, uint32_t qmeta_stride,
                      uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off, const uint32_t* item_off,
                      const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, uint8_t* q8, float* u, uint32_t* tau,
                      uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st);
// rabitq lists (1-bit codes, 4-bit queries): the expanded-bits contraction of prefilter_rb.hip over 128 pairs per item.
bool ivf_pq_supports(const vsag_amd_store* s);
uint32_t ivf_pq_pairs_per_item();
int launch_ivf_pq(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
                  const uint32_t* pair_off, const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound,
                  int32_t* tq, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const int32_t* buckets,
                  uint32_t* gpairs, uint32_t gpairs_cap, hipStream_t st);
bool ivf_rb_supports(const vsag_amd_store* s);
uint32_t ivf_rb_pairs_per_item();
uint32_t ivf_rb_chunk_tiles();
size_t ivf_rb_scratch_bytes(const vsag_amd_store* s, uint64_t nq);
int launch_ivf_rb(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
                  const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, uint8_t* scratch,
                  uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st);
int launch_ivf_clear_gated(uint32_t* gate, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t* partial_cnt,
                           const int32_t* buckets, uint32_t* gpairs, uint32_t gpairs_cap, uint32_t k, hipStream_t st);
bool ivf_h16_supports(const vsag_amd_store* s);
uint32_t ivf_h16_pairs_per_item();
size_t ivf_h16_scratch_bytes(const vsag_amd_store* s, uint64_t nq);
int launch_ivf_h16(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
                   const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, float* tau,
                   uint8_t* scratch, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, hipStream_t st);
bool ivf_f32_supports(const vsag_amd_store* s);
uint32_t ivf_f32_pairs_per_item();
int launch_ivf_f32(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, const uint32_t* pair_off,
                   const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound, uint32_t kcand, float* tau,
                   uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const float* res_term, hipStream_t st);
int launch_ivf_rescore(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
                       uint32_t per_pair, uint64_t* partial, uint32_t* partial_cnt, const uint32_t* bound,
                       const float* res_term, hipStream_t st);
int launch_ivf_i8(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t kcand,
                  const uint32_t* pair_off, const uint32_t* item_off, const uint32_t* sorted_pair, const uint32_t* bound,
                  int32_t* tq, uint64_t* partial, uint32_t* partial_cnt, uint32_t* gate, const int32_t* buckets,
                  uint32_t* gpairs, uint32_t gpairs_cap, hipStream_t st);
int prepare_queries(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, const QueryLayout& ql,
                    uint32_t* qtab, float* qmeta, uint8_t* qcodes, hipStream_t st);
ScanArgs make_scan_args(const vsag_amd_store* s, const QueryLayout& ql, const uint32_t* qtab, const float* qmeta);
void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);
int launch_residual_terms(const vsag_amd_store* s, const float* queries, uint64_t nq, const int32_t* buckets, uint32_t nprobe,
                          float* terms, hipStream_t st);
int launch_merge_partials(const uint64_t* partial, const uint32_t* partial_cnt, const uint32_t* bound, uint32_t nslots,
                          uint32_t stride, uint32_t k, uint32_t S, uint64_t nq, uint32_t* ids, float* dists,
                          hipStream_t st);

// Up to five word arrays set in one launch.
struct FillJob {
    uint32_t* p[5];
    uint32_t v[5];
    uint64_t n[5];
};

__global__ void
fill_jobs_kernel(FillJob j) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
#pragma unroll
    for (int a = 0; a < 5; ++a) {
        if (i < j.n[a]) {
            j.p[a][i] = j.v[a];
        }
    }
}

// Pairs of probe columns [p0, p1): how many queries probe each list.
__global__ void
count_pairs_kernel(const int32_t* buckets, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t p1, uint32_t nlist,
                   uint32_t* counts) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint32_t w = p1 - p0;
    if (i >= nq * w) {
        return;
    }
    uint64_t q = i / w;
    uint32_t p = p0 + static_cast<uint32_t>(i % w);
    int32_t b = buckets[q * nprobe + p];
    if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
        atomicAdd(&counts[b], 1U);
    }
}

// The same grouping for many pairs without an atomic per pair in global memory (hundreds of thousands of them on a
// few thousand counters take 0.1 ms per launch): a counting sort in three launches.  kRegroupGroups workgroups each
// take a run of the pairs; regroup_hist_kernel counts a run's pairs per list in LDS, regroup_prefix_kernel turns
// the counts of a list into the offsets of the runs inside the list (and their sum into counts[]), and
// regroup_scatter_kernel hands out the places of a run with a cursor per list in LDS.
constexpr uint32_t kRegroupGroups = 128;
constexpr uint32_t kRegroupLists = 8192;  // lists a workgroup's LDS holds a counter for

__global__ void __launch_bounds__(1024)
regroup_hist_kernel(const int32_t* buckets, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t p1, uint32_t nlist,
                    uint32_t* hist) {
    __shared__ uint32_t h[kRegroupLists];
    for (uint32_t b = threadIdx.x; b < nlist; b += blockDim.x) {
        h[b] = 0;
    }
    __syncthreads();
    const uint32_t w = p1 - p0;
    const uint64_t total = nq * w, per = (total + gridDim.x - 1) / gridDim.x;
    const uint64_t begin = blockIdx.x * per, end = begin + per < total ? begin + per : total;
    for (uint64_t i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const uint64_t q = i / w;
        const int32_t b = buckets[q * nprobe + p0 + static_cast<uint32_t>(i - q * w)];
        if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
            atomicAdd(&h[b], 1U);
        }
    }
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < nlist; b += blockDim.x) {
        hist[static_cast<uint64_t>(blockIdx.x) * nlist + b] = h[b];
    }
}

__global__ void __launch_bounds__(256)
regroup_prefix_kernel(uint32_t* hist, uint32_t groups, uint32_t nlist, uint32_t* counts) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nlist) {
        return;
    }
    uint32_t running = 0;
    // Sixteen loads in flight at a time (the stores into the same array would otherwise keep them apart).
    for (uint32_t g0 = 0; g0 < groups; g0 += 16) {
        uint32_t c[16];
#pragma unroll
        for (uint32_t u = 0; u < 16; ++u) {
            c[u] = g0 + u < groups ? hist[static_cast<uint64_t>(g0 + u) * nlist + b] : 0U;
        }
#pragma unroll
        for (uint32_t u = 0; u < 16; ++u) {
            if (g0 + u < groups) {
                hist[static_cast<uint64_t>(g0 + u) * nlist + b] = running;
                running += c[u];
            }
        }
    }
    counts[b] = running;
}

__global__ void __launch_bounds__(1024)
regroup_scatter_kernel(const int32_t* buckets, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t p1, uint32_t nlist,
                       const uint32_t* pair_off, const uint32_t* hist, uint32_t* sorted_pair) {
    __shared__ uint32_t cursor[kRegroupLists];
    for (uint32_t b = threadIdx.x; b < nlist; b += blockDim.x) {
        cursor[b] = 0;
    }
    __syncthreads();
    const uint32_t w = p1 - p0;
    const uint64_t total = nq * w, per = (total + gridDim.x - 1) / gridDim.x;
    const uint64_t begin = blockIdx.x * per, end = begin + per < total ? begin + per : total;
    for (uint64_t i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const uint64_t q = i / w;
        const uint32_t p = p0 + static_cast<uint32_t>(i - q * w);
        const int32_t b = buckets[q * nprobe + p];
        if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
            const uint32_t pos = pair_off[b] + hist[static_cast<uint64_t>(blockIdx.x) * nlist + b] + atomicAdd(&cursor[b], 1U);
            sorted_pair[pos] = static_cast<uint32_t>(q * nprobe + p);
        }
    }
}

// Chunks a list of `tiles` tiles is cut into: about tiles_per_item tiles each, at most chunks_max chunks
// (longer lists get longer chunks); 0xFFFFFFFF = never cut.
__device__ inline uint32_t
list_chunks(uint32_t tiles, uint32_t tiles_per_item, uint32_t chunks_max) {
    if (tiles_per_item == 0xFFFFFFFFU) {
        return tiles != 0 ? 1U : 0U;
    }
    uint32_t chunks = (tiles + tiles_per_item - 1) / tiles_per_item;
    return chunks < chunks_max ? chunks : chunks_max;
}

// Work items of a list: query groups x tile chunks.
__device__ inline uint32_t
list_items(uint32_t pairs, uint32_t T, uint32_t tiles, uint32_t tiles_per_item, uint32_t chunks_max) {
    return ((pairs + T - 1) / T) * list_chunks(tiles, tiles_per_item, chunks_max);
}

// Exclusive prefix sums of two per-thread values over a workgroup of up to 1024 threads; wave totals go
// through `wave_sums` (2 x 16 words of LDS).  Returns the grand totals.
__device__ inline void
block_exclusive_scan2(uint32_t& a, uint32_t& b, uint32_t (*wave_sums)[16], uint32_t& total_a, uint32_t& total_b) {
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6, nwaves = (blockDim.x + kWave - 1) >> 6;
    uint32_t ia = a, ib = b;
    for (int off = 1; off < kWave; off <<= 1) {
        uint32_t oa = __shfl_up(ia, off), ob = __shfl_up(ib, off);
        if (static_cast<int>(lane) >= off) {
            ia += oa;
            ib += ob;
        }
    }
    if (lane == kWave - 1) {
        wave_sums[0][wave] = ia;
        wave_sums[1][wave] = ib;
    }
    __syncthreads();
    uint32_t ba = 0, bb = 0;
    total_a = 0;
    total_b = 0;
    for (uint32_t w = 0; w < nwaves; ++w) {
        uint32_t sa = wave_sums[0][w], sb = wave_sums[1][w];
        if (w < wave) {
            ba += sa;
            bb += sb;
        }
        total_a += sa;
        total_b += sb;
    }
    a = ba + ia - a;
    b = bb + ib - b;
}

// One workgroup: exclusive prefix sums of the pair counts and of the work items.
__global__ void __launch_bounds__(1024)
offsets_kernel(const uint32_t* counts, const uint32_t* list_tile, uint32_t nlist, uint32_t T, uint32_t tiles_per_item,
               uint32_t chunks_max, uint32_t* pair_off, uint32_t* item_off) {
    __shared__ uint32_t wave_sums[2][16];
    uint32_t per = (nlist + blockDim.x - 1) / blockDim.x;
    uint32_t begin = threadIdx.x * per;
    uint32_t end = begin + per < nlist ? begin + per : nlist;
    uint32_t sp = 0, si = 0;
    for (uint32_t i = begin; i < end; ++i) {
        sp += counts[i];
        si += list_items(counts[i], T, list_tile[2 * i + 1] - list_tile[2 * i], tiles_per_item, chunks_max);
    }
    uint32_t rp = sp, ri = si, all_pairs, all_items;
    block_exclusive_scan2(rp, ri, wave_sums, all_pairs, all_items);
    if (threadIdx.x == 0) {
        pair_off[nlist] = all_pairs;
        item_off[nlist] = all_items;
    }
    for (uint32_t i = begin; i < end; ++i) {
        pair_off[i] = rp;
        item_off[i] = ri;
        rp += counts[i];
        ri += list_items(counts[i], T, list_tile[2 * i + 1] - list_tile[2 * i], tiles_per_item, chunks_max);
    }
}

__global__ void
scatter_pairs_kernel(const int32_t* buckets, uint64_t nq, uint32_t nprobe, uint32_t p0, uint32_t p1, uint32_t nlist,
                     const uint32_t* pair_off, uint32_t* cursor, uint32_t* sorted_pair) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint32_t w = p1 - p0;
    if (i >= nq * w) {
        return;
    }
    uint64_t q = i / w;
    uint32_t p = p0 + static_cast<uint32_t>(i % w);
    int32_t b = buckets[q * nprobe + p];
    if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
        uint32_t pos = pair_off[b] + atomicAdd(&cursor[b], 1U);
        sorted_pair[pos] = static_cast<uint32_t>(q * nprobe + p);
    }
}

// The three regrouping steps above for a small batch (all probe columns) in one workgroup.
__global__ void __launch_bounds__(1024)
regroup_small_kernel(const int32_t* buckets, uint64_t nq, uint32_t nprobe, const uint32_t* list_tile, uint32_t nlist,
                     uint32_t T, uint32_t tiles_per_item, uint32_t chunks_max, uint32_t* counts, uint32_t* cursor,
                     uint32_t* pair_off, uint32_t* item_off, uint32_t* sorted_pair) {
    __shared__ uint32_t wave_sums[2][16];
    const uint64_t npairs = nq * nprobe;
    for (uint32_t i = threadIdx.x; i <= nlist; i += blockDim.x) {
        counts[i] = 0;
        cursor[i] = 0;
    }
    __syncthreads();
    for (uint64_t i = threadIdx.x; i < npairs; i += blockDim.x) {
        int32_t b = buckets[i];
        if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
            atomicAdd(&counts[b], 1U);
        }
    }
    // The counts were made by atomics in L2; the fences keep the plain loads below from an older cached line.
    __threadfence();
    __syncthreads();
    __threadfence();
    uint32_t per = (nlist + blockDim.x - 1) / blockDim.x;
    uint32_t begin = threadIdx.x * per;
    uint32_t end = begin + per < nlist ? begin + per : nlist;
    uint32_t sp = 0, si = 0;
    for (uint32_t i = begin; i < end; ++i) {
        sp += counts[i];
        si += list_items(counts[i], T, list_tile[2 * i + 1] - list_tile[2 * i], tiles_per_item, chunks_max);
    }
    uint32_t rp = sp, ri = si, all_pairs, all_items;
    block_exclusive_scan2(rp, ri, wave_sums, all_pairs, all_items);
    if (threadIdx.x == 0) {
        pair_off[nlist] = all_pairs;
        item_off[nlist] = all_items;
    }
    for (uint32_t i = begin; i < end; ++i) {
        pair_off[i] = rp;
        item_off[i] = ri;
        rp += counts[i];
        ri += list_items(counts[i], T, list_tile[2 * i + 1] - list_tile[2 * i], tiles_per_item, chunks_max);
    }
    __syncthreads();
    for (uint64_t i = threadIdx.x; i < npairs; i += blockDim.x) {
        int32_t b = buckets[i];
        if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
            uint32_t pos = pair_off[b] + atomicAdd(&cursor[b], 1U);
            sorted_pair[pos] = static_cast<uint32_t>(i);
        }
    }
}

struct IvfArgs {
    const uint32_t* ids;         // inner id per tile slot
    const uint32_t* list_tile;   // 2 nlist: first tile and end of the used tiles of every list
    const uint32_t* pair_off;    // nlist+1
    const uint32_t* item_off;    // nlist+1
    const uint32_t* sorted_pair; // pair index (q * nprobe + p) grouped by list
    uint32_t nlist;
    uint32_t nprobe;
    uint32_t dummy_query;        // index of an all-zero query row
    uint32_t k;
    uint32_t S;
    const uint32_t* deny;        // filtered-out inner ids as a bit mask, or null
    uint32_t tiles_per_item;     // 0xFFFFFFFF: whole lists
    uint32_t chunks_max;         // partial lists per pair
    uint32_t* bound;             // per query: ordered distance no final candidate can exceed
    uint32_t* seed;              // nq x k first-tile minima by work-item class, or null (flat scan's cold start)
    uint64_t* partial;           // npairs_total x chunks_max x k keys
    uint32_t* partial_cnt;       // npairs_total x chunks_max
    const uint32_t* gate;        // per query, or null: only queries with a raised gate are served
    // Direct mode (non-null `direct`): the work is a short array of pairs instead of the per-list grouping;
    // direct_count[0] of them, each worth chunks_max consecutive items.  More than direct_cap pairs are left to a
    // launch over the grouping (which in turn stands back when direct mode can take them).
    const uint32_t* direct;
    const uint32_t* direct_count;
    uint32_t direct_cap;
    const int32_t* buckets;      // direct mode: list of a pair
    // Residual lists (bucket_datacell.h:553-566): the codes hold x - c of their list's centroid c, and a distance is
    // put right by taking off the slot's bias (l2: -2 <c, decoded> - |c|^2) and the pair's term (<q, c>, twice for l2).
    const float* res_bias;       // per slot, or null
    const float* res_term;       // per pair (q * nprobe + p), or null: no residual
};

constexpr uint32_t kIvfSeedTiles = 4;

// CHUNKED: work items are chunks of lists and start cold together (few queries); otherwise whole lists.
template <int KIND, int METRIC, int T, bool CHUNKED>
__device__ __forceinline__ void
ivf_scan_item(const ScanArgs& a, const IvfArgs& v, uint64_t* lds, uint32_t item) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint32_t list_begin, list_end, local, pfirst, plast;
    cu32_p pairs_src = as_const(v.sorted_pair);
    if (v.direct != nullptr) {
        const uint32_t count = as_const(v.direct_count)[0];
        const uint32_t vi = item / v.chunks_max;
        if (count > v.direct_cap || vi >= count) {
            return;
        }
        pairs_src = as_const(v.direct);
        const int32_t bk = v.buckets[pairs_src[vi]];  // a real list: pairs without one are never queued
        list_begin = as_const(v.list_tile)[2 * bk];
        list_end = as_const(v.list_tile)[2 * bk + 1];
        local = item % v.chunks_max;
        pfirst = vi;
        plast = vi + 1;
    } else {
        const uint32_t total = as_const(v.item_off)[v.nlist];
        if (item >= total) {
            return;
        }
        if (v.gate != nullptr) {
            // Words nq and nq + 1 of the gate array count the raised gates and their pairs: nothing to serve, or
            // few enough for the direct launch.
            const uint32_t raised = as_const(v.gate)[v.dummy_query];
            if (raised == 0 || (v.direct_cap != 0 && as_const(v.gate)[v.dummy_query + 1] <= v.direct_cap)) {
                return;
            }
        }
        // Which list: last b with item_off[b] <= item.
        cu32_p ioff = as_const(v.item_off);
        uint32_t lo = 0, hi = v.nlist;
        while (hi - lo > 1) {
            uint32_t mid = (lo + hi) >> 1;
            if (ioff[mid] <= item) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        list_begin = as_const(v.list_tile)[2 * lo];
        list_end = as_const(v.list_tile)[2 * lo + 1];
        local = item - ioff[lo];
        pfirst = as_const(v.pair_off)[lo];
        plast = as_const(v.pair_off)[lo + 1];
    }
    uint32_t group = local, chunk = 0;
    uint32_t tbeg = list_begin, tend = list_end;
    if (CHUNKED) {
        const uint32_t tiles = list_end - list_begin;
        const uint32_t chunks = list_chunks(tiles, v.tiles_per_item, v.chunks_max);
        if (chunks == 0) {
            return;
        }
        const uint32_t per = (tiles + chunks - 1) / chunks;
        chunk = group % chunks;
        group = group / chunks;
        tbeg = list_begin + chunk * per;
        tbeg = tbeg < list_end ? tbeg : list_end;
        tend = tbeg + per < list_end ? tbeg + per : list_end;
    }
    const uint32_t pbeg = pfirst + group * T;
    const uint32_t pend = plast;

    const uint32_t S = v.S, k = v.k;
    const uint32_t spend = selector_base(S, k);  // where a selector's pending keys start
    uint64_t* sel = lds + static_cast<size_t>(wave) * T * S;
    uint32_t qidx[T], pair[T];
    uint64_t tau[T];
    uint32_t cnt[T];
    uint32_t cold[T];  // tiles after which this item still looks at the seed row (see the flat scan)
    bool any_live = false;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        bool live = pbeg + t < pend;
        pair[t] = live ? pairs_src[pbeg + t] : 0xFFFFFFFFU;
        if (live && v.gate != nullptr && as_const(v.gate)[pair[t] / v.nprobe] == 0) {
            live = false;
            pair[t] = 0xFFFFFFFFU;
        }
        any_live = any_live || live;
        qidx[t] = live ? pair[t] / v.nprobe : v.dummy_query;
        cnt[t] = 0;
        uint32_t bound = live ? __builtin_amdgcn_readfirstlane(__atomic_load_n(&v.bound[qidx[t]], __ATOMIC_RELAXED))
                              : 0U;
        // Everything at or below the bound passes, whatever its id.
        tau[t] = (static_cast<uint64_t>(bound) << 32) | 0xFFFFFFFFULL;
        cold[t] = CHUNKED && v.seed != nullptr && live && bound == 0xFFFFFFFFU ? kIvfSeedTiles : 0;
    }
    if (!any_live) {
        return;  // nothing but gated-off queries
    }
    const uint32_t seed_slot = item % k;
    for (uint32_t i = lane; i < T * S; i += kWave) {
        sel[i] = kInfKey;
    }
    wave_lds_fence();

    const QueryRows<T> qrows = query_rows<T>(a, qidx);
    float rterm[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        rterm[t] = v.res_term != nullptr && pair[t] != 0xFFFFFFFFU ? v.res_term[pair[t]] : 0.0F;
    }
    constexpr int GROUP = GroupOf<T>::value;
    TileStream<GROUP> cur{a.tiles, lane, tbeg, tend, 1, 0, a.G};
    TileStream<GROUP> nxt = cur;
    uint4 buf_a[GROUP], buf_b[GROUP];
    if (cur.valid()) {
        cur.load(buf_a, cur.tile);
    }
    Acc<KIND, T> acc;
    acc_reset(acc);

    auto consume = [&](const uint4(&regs)[GROUP]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            if (cur.j0 + u < a.G) {
                accumulate_granule<KIND, METRIC, T>(a, qrows, cur.j0 + u, regs[u], acc);
            }
        }
        if (cur.j0 + GROUP < a.G) {
            return;
        }
        const uint64_t slot = cur.tile * kWave + lane;
        float d[T];
        finish_distances<KIND, METRIC, T>(a, qidx, slot, acc, d);
        acc_reset(acc);
        if (v.res_term != nullptr) {
            const float bias = v.res_bias != nullptr ? v.res_bias[slot] : 0.0F;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                d[t] = (d[t] - bias) - rterm[t];
            }
        }
        const uint32_t id = v.ids[slot];
        const bool valid = id != VSAG_AMD_INVALID_ID && !denied(v.deny, id);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint64_t key = make_key(d[t], id);
            if (CHUNKED && cold[t] != 0) {
                uint32_t* row = v.seed + static_cast<uint64_t>(qidx[t]) * k;
                if (cold[t] == kIvfSeedTiles) {
                    uint32_t m = wave_min_u32(valid ? static_cast<uint32_t>(key >> 32) : 0xFFFFFFFFU);
                    lower_shared(&row[seed_slot], m, lane);
                }
                --cold[t];
                uint32_t mx = 0;
                for (uint32_t i = lane; i < k; i += kWave) {
                    uint32_t sv = __atomic_load_n(&row[i], __ATOMIC_RELAXED);
                    mx = sv > mx ? sv : mx;
                }
                mx = wave_max_u32(mx);
                if (mx != 0xFFFFFFFFU) {
                    cold[t] = 0;
                    mx = lower_shared(&v.bound[qidx[t]], mx, lane);
                    uint64_t shared_tau = (static_cast<uint64_t>(mx) << 32) | 0xFFFFFFFFULL;
                    tau[t] = tau[t] < shared_tau ? tau[t] : shared_tau;
                }
            }
            bool pass = valid && key < tau[t];
            uint64_t mask = __ballot(pass);
            if (mask == 0) {
                continue;
            }
            uint64_t* keys = sel + t * S;
            uint32_t np = __popcll(mask);
            if (spend + cnt[t] + np > S) {
                uint64_t th = selector_flush(keys, S, k, cnt[t], lane);
                cnt[t] = 0;
                cold[t] = 0;
                if (pair[t] != 0xFFFFFFFFU) {
                    // th finite: this pair alone already holds k candidates at or below th.
                    uint32_t bound = lower_shared(&v.bound[qidx[t]], static_cast<uint32_t>(th >> 32), lane);
                    uint64_t shared_tau = (static_cast<uint64_t>(bound) << 32) | 0xFFFFFFFFULL;
                    tau[t] = th < shared_tau ? th : shared_tau;
                }
            }
            if (pass) {
                keys[spend + cnt[t] + mask_rank(mask)] = key;
            }
            cnt[t] += np;
        }
    };

    while (cur.valid()) {
        nxt.advance();
        nxt.load(buf_b, cur.tile);
        consume(buf_a);
        cur = nxt;
        if (!cur.valid()) {
            break;
        }
        nxt.advance();
        nxt.load(buf_a, cur.tile);
        consume(buf_b);
        cur = nxt;
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (pair[t] == 0xFFFFFFFFU) {
            continue;
        }
        // What the shared bound still admits is usually less than k keys, which go out unsorted; only a
        // pair left with more sorts once more (and then has a k-th key to lower the bound with).
        uint64_t* keys = sel + t * S;
        wave_lds_fence();
        uint32_t bs = __builtin_amdgcn_readfirstlane(__atomic_load_n(&v.bound[qidx[t]], __ATOMIC_RELAXED));
        uint32_t total = spend + cnt[t];
        uint32_t admitted = selector_count_admitted(keys, total, bs, lane);
        if (admitted > k) {
            uint64_t th = selector_flush(keys, S, k, cnt[t], lane);
            bs = lower_shared(&v.bound[qidx[t]], static_cast<uint32_t>(th >> 32), lane);
            total = k;
            admitted = selector_count_admitted(keys, total, bs, lane);
        } else if (admitted == k) {
            // Exactly k admitted keys: their largest distance is a bound other pairs can use.
            uint32_t mx = 0;
            for (uint32_t i = lane; i < total; i += kWave) {
                uint64_t key = keys[i];
                uint32_t od = static_cast<uint32_t>(key >> 32);
                mx = key != kInfKey && od <= bs && od > mx ? od : mx;
            }
            lower_shared(&v.bound[qidx[t]], wave_max_u32(mx), lane);  // bs itself must stay what was counted with
        }
        const uint64_t list = static_cast<uint64_t>(pair[t]) * v.chunks_max + chunk;
        if (lane == 0) {
            v.partial_cnt[list] = admitted;
        }
        if (admitted != 0) {
            selector_copy_admitted(keys, total, bs, v.partial + list * k, lane);
        }
    }
}

// A wave is a work item.  The direct launch (v.direct) serves a queue whose length only the device knows: a grid sized
// for its capacity would be tens of thousands of workgroups that find nothing to do, so there the waves of a smaller
// grid take the items in turn.
template <int KIND, int METRIC, int T, bool CHUNKED>
__global__ void __launch_bounds__(256)
ivf_scan_kernel(ScanArgs a, IvfArgs v) {
    extern __shared__ uint64_t lds[];
    const uint32_t waves = blockDim.x >> 6;
    uint32_t item = blockIdx.x * waves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (v.direct == nullptr) {
        ivf_scan_item<KIND, METRIC, T, CHUNKED>(a, v, lds, item);
        return;
    }
    const uint32_t count = as_const(v.direct_count)[0];
    const uint32_t stride = gridDim.x * waves;
    const uint32_t limit = count <= v.direct_cap ? count * v.chunks_max : 0;
    for (; item < limit; item += stride) {
        ivf_scan_item<KIND, METRIC, T, CHUNKED>(a, v, lds, item);
        // the selectors of the item in LDS have been read before the next item resets them
        wave_lds_fence();
    }
}

// Exact fp32 distances of the candidates of one query, best k kept.  One workgroup of four waves per query;
// sixteen lanes share a candidate, so a workgroup has sixteen gathered rows in flight.
constexpr uint32_t kRerankThreads = 256;

__global__ void __launch_bounds__(kRerankThreads)
rerank_kernel(const float* raw, uint64_t n, uint32_t dim, int metric, const float* queries, const uint32_t* cand,
              uint32_t kcand, uint32_t k, uint32_t S, uint32_t* ids, float* dists) {
    extern __shared__ uint64_t lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t sub = tid >> 4, l = tid & 15;  // candidate slot of this step, lane within it
    const uint64_t q = blockIdx.x;
    const float* qv = queries + q * dim;
    for (uint32_t i = tid; i < S; i += kRerankThreads) {
        lds[i] = kInfKey;
    }
    float inv_norm = 1.0F;
    if (metric == VSAG_AMD_METRIC_COSINE) {
        float s = 0.0F;
        for (uint32_t d = l; d < dim; d += 16) {
            s = fmaf(qv[d], qv[d], s);
        }
        for (int off = 8; off > 0; off >>= 1) {
            s += __shfl_xor(s, off);
        }
        inv_norm = s > 0.0F ? 1.0F / sqrtf(s) : 1.0F;
    }
    __syncthreads();
    const bool vec4 = (dim & 3) == 0;
    for (uint32_t j0 = 0; j0 < kcand; j0 += kRerankThreads / 16) {
        const uint32_t j = j0 + sub;
        uint32_t id = j < kcand ? as_const(cand)[q * kcand + j] : VSAG_AMD_INVALID_ID;
        const bool live = id != VSAG_AMD_INVALID_ID && id < n;
        const float* x = raw + static_cast<uint64_t>(live ? id : 0) * dim;
        float s = 0.0F, xx = 0.0F;
        if (live) {
            if (vec4) {
                for (uint32_t d = l * 4; d < dim; d += 64) {
                    float4 xv = *reinterpret_cast<const float4*>(x + d);
                    float4 qq = *reinterpret_cast<const float4*>(qv + d);
                    if (metric == VSAG_AMD_METRIC_L2) {
                        float t0 = qq.x - xv.x, t1 = qq.y - xv.y, t2 = qq.z - xv.z, t3 = qq.w - xv.w;
                        s = fmaf(t0, t0, s);
                        s = fmaf(t1, t1, s);
                        s = fmaf(t2, t2, s);
                        s = fmaf(t3, t3, s);
                    } else {
                        s = fmaf(qq.x, xv.x, s);
                        s = fmaf(qq.y, xv.y, s);
                        s = fmaf(qq.z, xv.z, s);
                        s = fmaf(qq.w, xv.w, s);
                        xx = fmaf(xv.x, xv.x, xx);
                        xx = fmaf(xv.y, xv.y, xx);
                        xx = fmaf(xv.z, xv.z, xx);
                        xx = fmaf(xv.w, xv.w, xx);
                    }
                }
            } else {
                for (uint32_t d = l; d < dim; d += 16) {
                    float xv = x[d];
                    if (metric == VSAG_AMD_METRIC_L2) {
                        float t = qv[d] - xv;
                        s = fmaf(t, t, s);
                    } else {
                        s = fmaf(qv[d], xv, s);
                        xx = fmaf(xv, xv, xx);
                    }
                }
            }
        }
        for (int off = 8; off > 0; off >>= 1) {
            s += __shfl_xor(s, off);
            xx += __shfl_xor(xx, off);
        }
        if (live && l == 0) {
            float dist;
            if (metric == VSAG_AMD_METRIC_L2) {
                dist = s;
            } else if (metric == VSAG_AMD_METRIC_IP) {
                dist = 1.0F - s;
            } else {
                float xn = xx > 0.0F ? 1.0F / sqrtf(xx) : 1.0F;
                dist = 1.0F - s * inv_norm * xn;
            }
            lds[j] = make_key(dist, id);
        }
    }
    __syncthreads();
    if (tid >= kWave) {
        return;
    }
    wave_bitonic_sort(lds, S, tid);
    for (uint32_t i = tid; i < k; i += kWave) {
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

// Exact fp32 distance of every (query, inner id) pair, in the order given: what the rerank computes for a candidate,
// without the selection.  Sixteen lanes share a pair; ids beyond the rows (or VSAG_AMD_INVALID_ID) give -1.
__global__ void __launch_bounds__(kRerankThreads)
rows_distances_kernel(const float* raw, uint64_t n, uint32_t dim, int metric, const float* queries, const uint32_t* ids,
                      uint32_t count, float* dists) {
    const uint32_t tid = threadIdx.x;
    const uint32_t sub = tid >> 4, l = tid & 15;
    const uint64_t q = blockIdx.y;
    const float* qv = queries + q * dim;
    float inv_norm = 1.0F;
    if (metric == VSAG_AMD_METRIC_COSINE) {
        float s = 0.0F;
        for (uint32_t d = l; d < dim; d += 16) {
            s = fmaf(qv[d], qv[d], s);
        }
        for (int off = 8; off > 0; off >>= 1) {
            s += __shfl_xor(s, off);
        }
        inv_norm = s > 0.0F ? 1.0F / sqrtf(s) : 1.0F;
    }
    const uint32_t j = blockIdx.x * (kRerankThreads / 16) + sub;
    const uint32_t id = j < count ? ids[q * count + j] : VSAG_AMD_INVALID_ID;
    const bool live = id != VSAG_AMD_INVALID_ID && id < n;
    const float* x = raw + static_cast<uint64_t>(live ? id : 0) * dim;
    float s = 0.0F, xx = 0.0F;
    if (live) {
        if ((dim & 3) == 0) {
            for (uint32_t d = l * 4; d < dim; d += 64) {
                const float4 xv = *reinterpret_cast<const float4*>(x + d);
                const float4 qq = *reinterpret_cast<const float4*>(qv + d);
                if (metric == VSAG_AMD_METRIC_L2) {
                    const float t0 = qq.x - xv.x, t1 = qq.y - xv.y, t2 = qq.z - xv.z, t3 = qq.w - xv.w;
                    s = fmaf(t0, t0, s);
                    s = fmaf(t1, t1, s);
                    s = fmaf(t2, t2, s);
                    s = fmaf(t3, t3, s);
                } else {
                    s = fmaf(qq.x, xv.x, s);
                    s = fmaf(qq.y, xv.y, s);
                    s = fmaf(qq.z, xv.z, s);
                    s = fmaf(qq.w, xv.w, s);
                    xx = fmaf(xv.x, xv.x, xx);
                    xx = fmaf(xv.y, xv.y, xx);
                    xx = fmaf(xv.z, xv.z, xx);
                    xx = fmaf(xv.w, xv.w, xx);
                }
            }
        } else {
            for (uint32_t d = l; d < dim; d += 16) {
                const float xv = x[d];
                if (metric == VSAG_AMD_METRIC_L2) {
                    const float t = qv[d] - xv;
                    s = fmaf(t, t, s);
                } else {
                    s = fmaf(qv[d], xv, s);
                    xx = fmaf(xv, xv, xx);
                }
            }
        }
    }
    for (int off = 8; off > 0; off >>= 1) {
        s += __shfl_xor(s, off);
        xx += __shfl_xor(xx, off);
    }
    if (j < count && l == 0) {
        float dist = -1.0F;
        if (live) {
            if (metric == VSAG_AMD_METRIC_L2) {
                dist = s;
            } else if (metric == VSAG_AMD_METRIC_IP) {
                dist = 1.0F - s;
            } else {
                const float xn = xx > 0.0F ? 1.0F / sqrtf(xx) : 1.0F;
                dist = 1.0F - s * inv_norm * xn;
            }
        }
        dists[q * count + j] = dist;
    }
}

template <int KIND, int METRIC, int T>
static void
launch_ivf_c(dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a, const IvfArgs& v) {
    if (v.tiles_per_item != 0xFFFFFFFFU) {
        hipLaunchKernelGGL((ivf_scan_kernel<KIND, METRIC, T, true>), grid, block, lds, st, a, v);
    } else {
        hipLaunchKernelGGL((ivf_scan_kernel<KIND, METRIC, T, false>), grid, block, lds, st, a, v);
    }
}

template <int KIND, int METRIC>
static void
launch_ivf_t(int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a, const IvfArgs& v) {
    switch (T) {
        case 1:
            launch_ivf_c<KIND, METRIC, 1>(grid, block, lds, st, a, v);
            break;
        case 2:
            launch_ivf_c<KIND, METRIC, 2>(grid, block, lds, st, a, v);
            break;
        default:
            launch_ivf_c<KIND, METRIC, 4>(grid, block, lds, st, a, v);
            break;
    }
}

template <int KIND>
static void
launch_ivf_m(int metric, int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a,
             const IvfArgs& v) {
    if (metric == VSAG_AMD_METRIC_L2) {
        launch_ivf_t<KIND, VSAG_AMD_METRIC_L2>(T, grid, block, lds, st, a, v);
    } else if (metric == VSAG_AMD_METRIC_COSINE && (KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32)) {
        launch_ivf_t<KIND, VSAG_AMD_METRIC_COSINE>(T, grid, block, lds, st, a, v);
    } else {
        launch_ivf_t<KIND, VSAG_AMD_METRIC_IP>(T, grid, block, lds, st, a, v);
    }
}

static int
launch_ivf(const vsag_amd_store* s, int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a,
           const IvfArgs& v) {
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
            launch_ivf_m<VSAG_AMD_KIND_FP32>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_SQ8:
            launch_ivf_m<VSAG_AMD_KIND_SQ8>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_SQ4:
            launch_ivf_m<VSAG_AMD_KIND_SQ4>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            launch_ivf_m<VSAG_AMD_KIND_SQ4_UNIFORM>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            launch_ivf_m<VSAG_AMD_KIND_SQ8_UNIFORM>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_PQFS:
            launch_ivf_m<VSAG_AMD_KIND_PQFS>(s->metric, T, grid, block, lds, st, a, v);
            break;
        case VSAG_AMD_KIND_RABITQ:
            if (s->query_bits == 32) {
                launch_ivf_m<kKindRabitqF32>(s->metric, T, grid, block, lds, st, a, v);
            } else {
                launch_ivf_m<VSAG_AMD_KIND_RABITQ>(s->metric, T, grid, block, lds, st, a, v);
            }
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

struct IvfBuffers {
    uint32_t* qtab;
    float* qmeta;
    uint8_t* qcodes;
    uint32_t* counts;     // nlist + 1
    uint32_t* cursor;     // nlist + 1
    uint32_t* pair_off;   // nlist + 1
    uint32_t* item_off;   // nlist + 1
    uint32_t* sorted_pair;
    uint32_t* hist;       // counting sort of many pairs: kRegroupGroups x nlist
    uint32_t* bound;
    uint32_t* seed;
    uint32_t* partial_cnt;
    uint64_t* partial;
    uint32_t* gate;       // mfma: nq + 3 (flags, raised gates, the pairs to scan again, the pairs queued)
    int32_t* tq;          // mfma: 2 (nq + 1)
    uint32_t* gpairs;     // mfma: pairs of gated queries, kGatedPairsCap
    uint8_t* q8;          // sq8 lists on the matrix cores: the planes of the queries, their scalars and thresholds
                          // (rabitq lists: the queries as bytes and their four factors)
    float* q8_u;
    uint32_t* q8_tau;
    float* res_term;      // residual lists: per pair
};

// Pairs of gated queries the direct fallback launch takes; more go through the per-list grouping.
constexpr uint32_t kGatedPairsCap = 32768;

static void
plan_ivf(const vsag_amd_store* s, uint64_t nq, uint32_t nprobe, uint32_t kcand, ScanPlanIvf* p) {
    p->S = selector_slots(kcand);
    uint64_t npairs = nq * nprobe;
    uint64_t avg = s->nlist ? npairs / s->nlist : 1;
    int t = 4;
    if (s->kind == VSAG_AMD_KIND_RABITQ || ((s->kind == VSAG_AMD_KIND_SQ8 || s->kind == VSAG_AMD_KIND_SQ4) &&
                                            s->metric == VSAG_AMD_METRIC_L2)) {
        t = 2;
    }
    while (t > 1 && static_cast<uint64_t>(t) > avg) {
        t >>= 1;
    }
    while (t > 1 && static_cast<size_t>(t) * p->S * 8 > 65536) {
        t >>= 1;
    }
    p->T = t;
    p->ql = query_layout(s);
    p->qcode_bytes = query_staging_bytes(s, nq);
    p->npairs = npairs;
    // Enough (list, query group) items to fill the machine: every item walks its whole list, the nearest list
    // of every query goes first.  Otherwise lists are cut into chunks of at least four tiles for about 4096 items in all (a probed
    // list is taken as twice the average length), at most 64 chunks per list and 256 MiB of partial lists.
    const uint64_t groups = div_up(npairs, static_cast<uint64_t>(t));
    p->chunked = groups < 8192 && s->max_list_tiles > 2;
    p->tiles_per_item = 0xFFFFFFFFU;
    p->chunks_max = 1;
    if (p->chunked) {
        const uint64_t avg_tiles = std::max<uint64_t>(1, s->nlist ? s->ntiles / s->nlist : 1);
        const uint64_t tpi = std::max<uint64_t>(4, div_up(groups * avg_tiles * 2, 4096));
        uint64_t cap = std::min<uint64_t>(64, div_up(s->max_list_tiles, tpi));
        while (cap > 1 && npairs * cap * kcand * 8 > (256ull << 20)) {
            cap /= 2;
        }
        p->tiles_per_item = static_cast<uint32_t>(std::min<uint64_t>(tpi, 0x7FFFFFFFU));
        p->chunks_max = static_cast<uint32_t>(cap);
    }
    p->seeded = p->chunked && kcand <= 256;
    // Large batches on sq4_uniform (and sq8_uniform / l2) lists: the streaming kernel scans the nearest list of every query, the int8
    // matrix cores the other columns, into two private lists per (query, list) pair.
    p->mfma = !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 && ivf_i8_supports(s) &&
              s->residual_centroids_dev == nullptr &&
              npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    // sq8 lists of at most 128 dimensions: the same split with the two-plane test and an exact rescoring.
    p->planes = !p->mfma && !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 && ivf_sq8_i8_supports(s) &&
                kcand <= ivf_rescore_capacity() && npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    p->bits1 = !p->mfma && !p->planes && !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 && ivf_rb_supports(s) &&
               kcand <= ivf_rescore_capacity() && npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    p->pq = !p->mfma && !p->planes && !p->bits1 && !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 &&
            ivf_pq_supports(s) && s->residual_centroids_dev == nullptr &&
            npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    // sq8 lists of more than 128 dimensions: the fp16 matrix cores (mode 2 keeps the fp32 ones; residual lists too).
    p->h16 = !p->mfma && !p->planes && !p->bits1 && !p->pq && !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 &&
             (scan_contraction_mode(s) != 2 || s->kind == VSAG_AMD_KIND_SQ4) && ivf_h16_supports(s) &&
             kcand <= ivf_rescore_capacity() &&
             npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    // fp32 lists, sq8 lists the fp16 pass does not take: the fp32 matrix cores pre-select, the same exact rescoring.
    p->f32 = !p->h16 && !p->mfma && !p->planes && !p->bits1 && !p->pq && !p->chunked && nprobe > 1 && scan_contraction_mode(s) >= 0 &&
             ivf_f32_supports(s) && kcand <= ivf_rescore_capacity() &&
             npairs * ivf_i8_lists_per_pair() * kcand * 8 <= (8ull << 30);
    p->mfma = p->mfma || p->planes || p->bits1 || p->pq || p->h16 || p->f32;
    if (p->mfma) {
        p->chunks_max = ivf_i8_lists_per_pair();
    }
}

// Whether the pairs of a call are grouped by the counting sort (regroup_hist_kernel ...) rather than with an atomic
// per pair.
static bool
regroup_by_sort(const vsag_amd_store* s, uint64_t npairs) {
    return npairs >= 65536 && s->nlist <= kRegroupLists;
}

static size_t
carve_ivf(Carver& c, const vsag_amd_store* s, const ScanPlanIvf& p, uint64_t nq, uint32_t kcand, IvfBuffers* b) {
    b->qtab = c.take<uint32_t>((nq + 1) * p.ql.qstride);
    b->qmeta = c.take<float>((nq + 1) * p.ql.qmeta);
    b->qcodes = c.take<uint8_t>(p.qcode_bytes);
    b->counts = c.take<uint32_t>(s->nlist + 1);
    b->cursor = c.take<uint32_t>(s->nlist + 1);
    b->pair_off = c.take<uint32_t>(s->nlist + 1);
    b->item_off = c.take<uint32_t>(s->nlist + 1);
    b->sorted_pair = c.take<uint32_t>(p.npairs);
    b->hist = c.take<uint32_t>(regroup_by_sort(s, p.npairs) ? static_cast<size_t>(kRegroupGroups) * s->nlist : 0);
    b->bound = c.take<uint32_t>(nq);
    b->seed = c.take<uint32_t>(p.seeded ? nq * kcand : 0);
    b->partial_cnt = c.take<uint32_t>(p.npairs * p.chunks_max);
    b->partial = c.take<uint64_t>(p.npairs * p.chunks_max * kcand);
    b->gate = c.take<uint32_t>(p.mfma ? nq + 3 : 0);
    b->gpairs = c.take<uint32_t>(p.mfma ? kGatedPairsCap : 0);
    b->tq = c.take<int32_t>(p.mfma ? 2 * (nq + 1) : 0);  // thresholds, then (sq8_uniform) the sums of the query values
    b->q8 = c.take<uint8_t>(p.planes ? ivf_sq8_i8_query_bytes(nq) : p.bits1 ? ivf_rb_scratch_bytes(s, nq)
                            : p.h16  ? ivf_h16_scratch_bytes(s, nq) : 0);
    b->q8_u = c.take<float>(p.planes ? ivf_sq8_i8_scalar_floats(nq) : 0);
    b->q8_tau = c.take<uint32_t>(p.planes ? ivf_sq8_i8_tau_words(nq) : 0);
    b->res_term = c.take<float>(s->residual_centroids_dev != nullptr ? p.npairs : 0);
    return c.used;
}

static int
check_ivf(const vsag_amd_store* s, uint64_t nq, uint32_t nprobe, uint32_t kcand) {
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(s->nlist > 0, "ivf scan on a flat store");
    VA_CHECK_ARG(kcand >= 1 && kcand <= kMaxTopK, "kcand must be in [1, %u], got %u", kMaxTopK, kcand);
    VA_CHECK_ARG(nprobe >= 1 && nprobe <= 65536, "nprobe must be in [1, 65536], got %u", nprobe);
    VA_CHECK_ARG(nq >= 1 && nq * nprobe < 0xFFFFFFFFull, "nq * nprobe must be below 2^32 - 1");
    return 0;
}

static inline uint32_t
blocks_for(uint64_t n) {
    return static_cast<uint32_t>(div_up(n ? n : 1, 256));
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_ivf_route_workspace_bytes(const vsag_amd_store_t* centroids, uint64_t nq, uint32_t nprobe) {
    return vsag_amd_flat_scan_workspace_bytes(centroids, nq, nprobe);
}

extern "C" int
vsag_amd_ivf_route(const vsag_amd_store_t* centroids, const float* queries_dev, uint64_t nq, uint32_t nprobe,
                   int32_t* buckets_dev, float* dists_dev, void* workspace_dev, size_t workspace_bytes, void* stream) {
    VA_CHECK_ARG(centroids != nullptr && centroids->kind == VSAG_AMD_KIND_FP32,
                 "routing needs an fp32 store of centroids");
    // VSAG_AMD_INVALID_ID and -1 are the same 32 bits, so the id buffer is the bucket buffer.
    return vsag_amd_flat_scan_topk(centroids, queries_dev, nq, nprobe, reinterpret_cast<uint32_t*>(buckets_dev),
                                   dists_dev, workspace_dev, workspace_bytes, stream);
}

extern "C" size_t
vsag_amd_ivf_scan_workspace_bytes(const vsag_amd_store_t* s, uint64_t nq, uint32_t nprobe, uint32_t kcand) {
    if (check_ivf(s, nq, nprobe, kcand) != 0) {
        return 0;
    }
    ScanPlanIvf p;
    plan_ivf(s, nq, nprobe, kcand, &p);
    Carver c(nullptr, 0);
    IvfBuffers b;
    return carve_ivf(c, s, p, nq, kcand, &b) + 256;
}

extern "C" int
vsag_amd_ivf_scan_topk(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, const int32_t* buckets_dev,
                       uint32_t nprobe, uint32_t kcand, uint32_t* ids_dev, float* dists_dev, void* workspace_dev,
                       size_t workspace_bytes, void* stream) {
    return vsag_amd_ivf_scan_topk_ex(s, queries_dev, nq, buckets_dev, nprobe, kcand, nullptr, ids_dev, dists_dev,
                                     workspace_dev, workspace_bytes, stream);
}

extern "C" int
vsag_amd_ivf_scan_topk_ex(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, const int32_t* buckets_dev,
                          uint32_t nprobe, uint32_t kcand, const vsag_amd_search_options_t* options, uint32_t* ids_dev,
                          float* dists_dev, void* workspace_dev, size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_ivf(s, nq, nprobe, kcand));
    VA_CHECK_ARG(queries_dev && buckets_dev && ids_dev && dists_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    ScanPlanIvf p;
    plan_ivf(s, nq, nprobe, kcand, &p);
    Carver c(workspace_dev, workspace_bytes);
    IvfBuffers b;
    carve_ivf(c, s, p, nq, kcand, &b);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);

    // Row nq of the query tables is the all-zero row that idle slots of a query tile point at.
    VA_TRY(prepare_queries(s, queries_dev, nq, nq + 1, p.ql, b.qtab, b.qmeta, b.qcodes, st));
    ScanArgs a = make_scan_args(s, p.ql, b.qtab, b.qmeta);
    const uint64_t nlists1 = static_cast<uint64_t>(s->nlist) + 1;
    const uint64_t nslots_all = p.npairs * p.chunks_max;
    const uint64_t nseed = p.seeded ? nq * kcand : 0;
    auto fill = [&](const FillJob& job) {
        uint64_t most = 0;
        for (uint64_t n : job.n) {
            most = std::max(most, n);
        }
        hipLaunchKernelGGL(fill_jobs_kernel, dim3(blocks_for(most)), dim3(256), 0, st, job);
    };
    fill(FillJob{{b.bound, b.partial_cnt, b.counts, b.cursor, b.seed},
                 {initial_bound(options), 0U, 0U, 0U, 0xFFFFFFFFU},
                 {nq, nslots_all, p.chunked ? 0 : nlists1, p.chunked ? 0 : nlists1, nseed}});

    IvfArgs v{};
    v.ids = s->ids_dev;
    v.list_tile = s->list_tile_dev;
    v.pair_off = b.pair_off;
    v.item_off = b.item_off;
    v.sorted_pair = b.sorted_pair;
    v.nlist = s->nlist;
    v.nprobe = nprobe;
    v.dummy_query = static_cast<uint32_t>(nq);
    v.k = kcand;
    v.S = p.S;
    v.deny = options != nullptr ? options->deny_bits_dev : nullptr;
    v.tiles_per_item = p.tiles_per_item;
    v.chunks_max = p.chunks_max;
    v.bound = b.bound;
    v.seed = p.seeded ? b.seed : nullptr;
    v.partial = b.partial;
    v.partial_cnt = b.partial_cnt;
    if (s->residual_centroids_dev != nullptr) {
        VA_TRY(launch_residual_terms(s, queries_dev, nq, buckets_dev, nprobe, b.res_term, st));
        v.res_term = b.res_term;
        v.res_bias = s->residual_bias_dev;
    }

    uint32_t waves = 4;
    while (waves > 1 && static_cast<size_t>(waves) * p.T * p.S * 8 > 65536) {
        waves >>= 1;
    }
    size_t lds = static_cast<size_t>(waves) * p.T * p.S * 8;
    // Whole lists: two passes, the nearest list of every query first (it seeds the per-query bound), then the
    // rest.  Chunked lists: all probe columns at once.
    uint32_t cols[3] = {0, p.chunked ? nprobe : 1, nprobe};
    // A pre-filter or a radius goes the streaming way (the matrix-core pass knows neither).
    const bool mfma = p.mfma && (options == nullptr || (options->deny_bits_dev == nullptr && options->use_radius == 0));
    // The pairs of columns [c0, c1) grouped by list (pair_off, sorted_pair) and the work items of every list (item_off).
    auto regroup = [&](uint32_t c0, uint32_t c1, uint64_t pairs, uint32_t per_item, uint32_t tiles_per_item,
                       uint32_t chunks_max) {
        if (b.hist != nullptr && pairs >= 65536) {
            hipLaunchKernelGGL(regroup_hist_kernel, dim3(kRegroupGroups), dim3(1024), 0, st, buckets_dev, nq, nprobe, c0,
                               c1, s->nlist, b.hist);
            hipLaunchKernelGGL(regroup_prefix_kernel, dim3(static_cast<uint32_t>(div_up(s->nlist, 256))), dim3(256), 0, st,
                               b.hist, kRegroupGroups, s->nlist, b.counts);
            hipLaunchKernelGGL(offsets_kernel, dim3(1), dim3(1024), 0, st, b.counts, s->list_tile_dev, s->nlist, per_item,
                               tiles_per_item, chunks_max, b.pair_off, b.item_off);
            hipLaunchKernelGGL(regroup_scatter_kernel, dim3(kRegroupGroups), dim3(1024), 0, st, buckets_dev, nq, nprobe,
                               c0, c1, s->nlist, b.pair_off, b.hist, b.sorted_pair);
            return;
        }
        hipLaunchKernelGGL(count_pairs_kernel, dim3(blocks_for(pairs)), dim3(256), 0, st, buckets_dev, nq, nprobe, c0, c1,
                           s->nlist, b.counts);
        hipLaunchKernelGGL(offsets_kernel, dim3(1), dim3(1024), 0, st, b.counts, s->list_tile_dev, s->nlist, per_item,
                           tiles_per_item, chunks_max, b.pair_off, b.item_off);
        hipLaunchKernelGGL(scatter_pairs_kernel, dim3(blocks_for(pairs)), dim3(256), 0, st, buckets_dev, nq, nprobe, c0,
                           c1, s->nlist, b.pair_off, b.cursor, b.sorted_pair);
    };
    timing_begin(st);
    for (int pass = 0; pass < 2; ++pass) {
        uint32_t p0 = cols[pass], p1 = cols[pass + 1];
        if (p1 <= p0) {
            continue;
        }
        uint64_t pairs = nq * (p1 - p0);
        if (pass == 1) {
            fill(FillJob{{b.counts, b.cursor, mfma ? b.gate : nullptr, nullptr, nullptr}, {0U, 0U, 0U, 0U, 0U},
                         {nlists1, nlists1, mfma ? nq + 3 : 0, 0, 0}});
        }
        if (pass == 1 && mfma) {
            // Pairs grouped by list once; workgroups of 256 pairs for the matrix cores, then -- for the queries whose
            // lists overflowed -- the streaming kernel's items over the same grouping.
            // ivf_i8.hip: items of 256 pairs, kIvfI8ChunkTiles, kIvfI8Chunks
            regroup(p0, p1, pairs,
                    p.bits1 ? ivf_rb_pairs_per_item() : p.pq ? ivf_pq_pairs_per_item() : p.h16 ? ivf_h16_pairs_per_item()
                    : p.f32 ? ivf_f32_pairs_per_item() : 256U,
                    p.bits1 ? ivf_rb_chunk_tiles() : 32U, 4U);
            if (p.h16) {
                VA_TRY(launch_ivf_h16(s, a, nq, nprobe, p0, b.pair_off, b.item_off, b.sorted_pair, b.bound, kcand,
                                      reinterpret_cast<float*>(b.tq), b.q8, b.partial, b.partial_cnt, b.gate, st));
                VA_TRY(launch_ivf_clear_gated(b.gate, nq, nprobe, p0, b.partial_cnt, buckets_dev, b.gpairs,
                                              kGatedPairsCap, kcand, st));
                VA_TRY(launch_ivf_rescore(s, a, nq, nprobe, p0, kcand, p.chunks_max, b.partial, b.partial_cnt, b.bound,
                                          nullptr, st));
            } else if (p.f32) {
                VA_TRY(launch_ivf_f32(s, a, nq, nprobe, p0, b.pair_off, b.item_off, b.sorted_pair, b.bound, kcand,
                                      reinterpret_cast<float*>(b.tq), b.partial, b.partial_cnt, b.gate, v.res_term, st));
                VA_TRY(launch_ivf_clear_gated(b.gate, nq, nprobe, p0, b.partial_cnt, buckets_dev, b.gpairs,
                                              kGatedPairsCap, kcand, st));
                VA_TRY(launch_ivf_rescore(s, a, nq, nprobe, p0, kcand, p.chunks_max, b.partial, b.partial_cnt, b.bound,
                                          v.res_term, st));
            } else if (p.pq) {
                VA_TRY(launch_ivf_pq(s, a, nq, nprobe, p0, kcand, b.pair_off, b.item_off, b.sorted_pair, b.bound, b.tq,
                                     b.partial, b.partial_cnt, b.gate, buckets_dev, b.gpairs, kGatedPairsCap, st));
            } else if (p.bits1) {
                VA_TRY(launch_ivf_rb(s, a, nq, nprobe, p0, b.pair_off, b.item_off, b.sorted_pair, b.bound, kcand, b.q8,
                                     b.partial, b.partial_cnt, b.gate, st));
                VA_TRY(launch_ivf_clear_gated(b.gate, nq, nprobe, p0, b.partial_cnt, buckets_dev, b.gpairs,
                                              kGatedPairsCap, kcand, st));
                VA_TRY(launch_ivf_rescore(s, a, nq, nprobe, p0, kcand, p.chunks_max, b.partial, b.partial_cnt, b.bound,
                                          nullptr, st));
            } else if (p.planes) {
                VA_TRY(launch_ivf_sq8_i8(s, reinterpret_cast<const float*>(a.qtab), a.qstride, a.qmeta, a.qmeta_stride, nq,
                                         nprobe, p0, b.pair_off, b.item_off, b.sorted_pair, b.bound, kcand, b.q8, b.q8_u,
                                         b.q8_tau, b.partial, b.partial_cnt, b.gate, st));
                VA_TRY(launch_ivf_clear_gated(b.gate, nq, nprobe, p0, b.partial_cnt, buckets_dev, b.gpairs,
                                              kGatedPairsCap, kcand, st));
                VA_TRY(launch_ivf_rescore(s, a, nq, nprobe, p0, kcand, p.chunks_max, b.partial, b.partial_cnt, b.bound,
                                          nullptr, st));
            } else {
                VA_TRY(launch_ivf_i8(s, a, nq, nprobe, p0, kcand, b.pair_off, b.item_off, b.sorted_pair, b.bound, b.tq,
                                     b.partial, b.partial_cnt, b.gate, buckets_dev, b.gpairs, kGatedPairsCap, st));
            }
            // Few gated pairs (the usual case): one wave per pair and chunk of its list.
            IvfArgs d = v;
            d.direct = b.gpairs;
            d.direct_count = b.gate + nq + 1;
            d.direct_cap = kGatedPairsCap;
            d.buckets = buckets_dev;
            d.tiles_per_item = 16;
            uint32_t dwaves = 4;
            while (dwaves > 1 && static_cast<size_t>(dwaves) * p.S * 8 > 65536) {
                dwaves >>= 1;
            }
            // (the waves of this grid take the queued items in turn: see ivf_scan_kernel)
            dim3 dgrid(static_cast<uint32_t>(std::min<uint64_t>(div_up(static_cast<uint64_t>(kGatedPairsCap) * d.chunks_max, dwaves),
                                                                8ull * static_cast<uint64_t>(device_cu_count()))));
            VA_TRY(launch_ivf(s, 1, dgrid, dim3(dwaves * kWave), static_cast<size_t>(dwaves) * p.S * 8, st, a, d));
            // Many: the streaming kernel's items over the same grouping (stands back otherwise).
            hipLaunchKernelGGL(offsets_kernel, dim3(1), dim3(1024), 0, st, b.counts, s->list_tile_dev, s->nlist,
                               static_cast<uint32_t>(p.T), 0xFFFFFFFFU, 1U, b.pair_off, b.item_off);
            v.gate = b.gate;
            v.direct_cap = kGatedPairsCap;
            uint64_t max_items = div_up(pairs, p.T) + std::min<uint64_t>(s->nlist, pairs);
            dim3 grid(static_cast<uint32_t>(div_up(max_items, waves)));
            VA_TRY(launch_ivf(s, p.T, grid, dim3(waves * kWave), lds, st, a, v));
            continue;
        }
        // The nearest-list pass ahead of the matrix cores: a list several times the average length (k-means leaves
        // such lists) would keep one wave busy long after the others are done, so lists are cut into chunks of about
        // the average list's length; a pair's chunks use the private lists the matrix-core pass has per pair anyway.
        IvfArgs first = v;
        const bool cut_first = mfma && pass == 0;
        // That pass lives on its selectors (no bound to start from), not on the list bytes: two queries per wave
        // instead of four mean twice the waves to overlap the flushes of each other (10M x 128, 64 lists: 0.59 ->
        // 0.45 ms).
        const int t_pass = cut_first ? std::min(p.T, 2) : p.T;
        if (cut_first) {
            const uint32_t avg_tiles = std::max<uint32_t>(1, static_cast<uint32_t>(s->ntiles / s->nlist));
            first.tiles_per_item = std::max<uint32_t>(std::max<uint32_t>(16, avg_tiles + avg_tiles / 4),
                                                      static_cast<uint32_t>(div_up(s->max_list_tiles, p.chunks_max)));
        }
        if (p.chunked) {
            hipLaunchKernelGGL(regroup_small_kernel, dim3(1), dim3(1024), 0, st, buckets_dev, nq, nprobe,
                               s->list_tile_dev, s->nlist, static_cast<uint32_t>(p.T), p.tiles_per_item, p.chunks_max,
                               b.counts, b.cursor, b.pair_off, b.item_off, b.sorted_pair);
        } else {
            regroup(p0, p1, pairs, static_cast<uint32_t>(t_pass), first.tiles_per_item, p.chunks_max);
        }
        // At most one partly filled query group per probed list, each cut into at most chunks_max items.
        uint64_t max_items =
            (div_up(pairs, t_pass) + std::min<uint64_t>(s->nlist, pairs)) * (p.chunked || cut_first ? p.chunks_max : 1);
        dim3 grid(static_cast<uint32_t>(div_up(max_items, waves)));
        VA_TRY(launch_ivf(s, t_pass, grid, dim3(waves * kWave), static_cast<size_t>(waves) * t_pass * p.S * 8, st, a, first));
    }
    if (!mfma) {
        timing_end(st);  // the matrix-core pass is timed on its own (ivf_i8.hip)
    }
    note_last_scan(mfma ? 256 : p.T, 0, 0);
    return launch_merge_partials(b.partial, b.partial_cnt, b.bound, nprobe * p.chunks_max, nprobe * p.chunks_max, kcand,
                                 p.S, nq, ids_dev, dists_dev, st);
}

namespace vsag_amd {
// Codes in the lists the queries probe, summed over all (query, probe) pairs.
__global__ void __launch_bounds__(256)
probed_codes_kernel(const int32_t* buckets, uint64_t npairs, uint32_t nlist, const uint32_t* list_sizes,
                    unsigned long long* total) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    unsigned long long mine = 0;
    if (i < npairs) {
        const int32_t b = buckets[i];
        if (b >= 0 && static_cast<uint32_t>(b) < nlist) {
            mine = list_sizes[b];
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        mine += __shfl_xor(mine, off);
    }
    if ((threadIdx.x & 63) == 0 && mine != 0) {
        atomicAdd(total, mine);
    }
}
}  // namespace vsag_amd

extern "C" int
vsag_amd_ivf_probed_codes(const vsag_amd_store_t* s, const int32_t* buckets_dev, uint64_t nq, uint32_t nprobe,
                          uint64_t* total_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(s != nullptr && s->nlist > 0, "not a posting-list store");
    VA_CHECK_ARG(buckets_dev && total_dev, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(fill_jobs_kernel, dim3(1), dim3(256), 0, st,
                       FillJob{{reinterpret_cast<uint32_t*>(total_dev), nullptr, nullptr, nullptr, nullptr}, {0, 0, 0, 0, 0},
                               {2, 0, 0, 0, 0}});
    hipLaunchKernelGGL(probed_codes_kernel, dim3(blocks_for(nq * nprobe)), dim3(256), 0, st, buckets_dev, nq * nprobe,
                       s->nlist, s->list_sizes_dev, reinterpret_cast<unsigned long long*>(total_dev));
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_rerank_fp32(const float* raw_dev, uint64_t n, uint32_t dim, int metric, const float* queries_dev, uint64_t nq,
                     const uint32_t* cand_ids_dev, uint32_t kcand, uint32_t k, uint32_t* ids_dev, float* dists_dev,
                     void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(raw_dev && queries_dev && cand_ids_dev && ids_dev && dists_dev, "null pointer");
    VA_CHECK_ARG(kcand >= 1 && kcand <= 4096, "kcand must be in [1, 4096], got %u", kcand);
    VA_CHECK_ARG(k >= 1 && k <= kcand, "k must be in [1, kcand], got %u", k);
    VA_CHECK_ARG(metric >= VSAG_AMD_METRIC_L2 && metric <= VSAG_AMD_METRIC_COSINE, "unknown metric %d", metric);
    VA_CHECK_ARG(nq >= 1 && nq < (1ull << 31), "nq must be in [1, 2^31)");
    uint32_t S = 64;
    while (S < kcand) {
        S <<= 1;
    }
    hipLaunchKernelGGL(rerank_kernel, dim3(static_cast<uint32_t>(nq)), dim3(kRerankThreads), S * 8,
                       static_cast<hipStream_t>(stream), raw_dev, n, dim, metric, queries_dev, cand_ids_dev, kcand, k,
                       S, ids_dev, dists_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" int
vsag_amd_rows_distances_fp32(const float* raw_dev, uint64_t n, uint32_t dim, int metric, const float* queries_dev,
                             uint64_t nq, const uint32_t* ids_dev, uint32_t count, float* dists_dev, void* stream) {
    VA_TRY(ensure_init());
    VA_CHECK_ARG(raw_dev && queries_dev && ids_dev && dists_dev, "null pointer");
    VA_CHECK_ARG(metric >= VSAG_AMD_METRIC_L2 && metric <= VSAG_AMD_METRIC_COSINE, "unknown metric %d", metric);
    VA_CHECK_ARG(nq >= 1 && nq <= 65535, "nq must be in [1, 65535]");
    VA_CHECK_ARG(count >= 1, "count must be positive");
    hipLaunchKernelGGL(rows_distances_kernel, dim3(static_cast<uint32_t>(div_up(count, kRerankThreads / 16)), static_cast<uint32_t>(nq)),
                       dim3(kRerankThreads), 0, static_cast<hipStream_t>(stream), raw_dev, n, dim, metric, queries_dev,
                       ids_dev, count, dists_dev);
    VA_HIP(hipGetLastError());
    return 0;
}
