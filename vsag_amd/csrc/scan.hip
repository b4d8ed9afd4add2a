// Flat scan with fused per-query top-k (BruteForce::SearchWithRequest hot loop,
// src/algorithm/bruteforce/bruteforce.cpp:481-597; FlattenDataCell::query,
// src/datacell/flatten_datacell.h:334-440), batched over queries.
//
// Work decomposition.  Grid x = query tile (T queries), y = chunk of code tiles.  A workgroup has up to
// four waves; wave w walks tiles chunk_begin + w, + W, ... with the next granule group already in flight,
// and keeps one LDS selector per query of the tile.  Workgroups that are resident together have
// consecutive x and the same y, so they stream the same chunk of codes at about the same time.
//
// Selection.  Every (wave, query) has a selector in LDS (topk.h).  Chunks and waves of one query share a
// per-query bound in global memory (the k-th best distance any of them has proven so far), so later
// work drops almost everything with one compare.  Each (chunk, wave) leaves a short counted list of the
// survivors that the bound still admits; a merge kernel picks the k best per query.  All waves of a query
// share a handful of addresses (its bound, its seed row), and atomics on one address serialise in L2, so
// every atomicMin is preceded by a plain load and issued only when it would lower the value.
#include <atomic>
#include <mutex>

#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);
int prepare_queries(const vsag_amd_store* s, const float* queries, uint64_t nq, uint64_t nq_pad, const QueryLayout& ql,
                    uint32_t* qtab, float* qmeta, uint8_t* qcodes, hipStream_t st);
ScanArgs make_scan_args(const vsag_amd_store* s, const QueryLayout& ql, const uint32_t* qtab, const float* qmeta);
uint64_t rabitq_query_code_size(uint32_t dim, int metric, int query_bits);

constexpr uint32_t kMaxWaves = 4;

// Zeroes two word arrays.
__global__ void
fill_words2_kernel(uint32_t* a, uint64_t na, uint32_t* b, uint64_t nb) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < na) {
        a[i] = 0;
    }
    if (i < nb) {
        b[i] = 0;
    }
}

// bound[q] = the k-th distance of a merged result, when there is one.
__global__ void
tighten_bound_kernel(const float* dists, uint32_t k, uint64_t nq, uint32_t* bound) {
    uint64_t q = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q < nq) {
        float kth = dists[q * k + k - 1];
        if (kth < __builtin_inff()) {
            uint32_t o = float_to_ordered(kth);
            if (o < bound[q]) {
                bound[q] = o;
            }
        }
    }
}

// Per query: no bound yet, no seeds yet.
__global__ void
reset_queries_kernel(uint32_t* bound, uint32_t bound0, uint64_t nq, uint32_t* seed, uint64_t nseed) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < nq) {
        bound[i] = bound0;
    }
    if (i < nseed) {
        seed[i] = 0xFFFFFFFFU;
    }
}

struct FlatArgs {
    uint64_t n;
    uint64_t tile0;         // the launch covers tiles [tile0, tile_end)
    uint64_t tile_end;
    uint64_t tiles_per_chunk;
    uint64_t nq;
    uint32_t k;
    uint32_t S;
    uint32_t nslots;        // partial lists per query (all launches of the call)
    uint32_t slot0;         // first list of this launch
    const uint32_t* gate;   // per query: 0 = this launch leaves the query alone; null = every query
    uint32_t* bound;        // per query: ordered distance that k candidates are known to reach
    uint64_t* partial;      // nq x nslots x k keys
    uint32_t* partial_cnt;  // nq x nslots
    uint32_t* seed;         // nq x k smallest first-tile distances by wave class, or null (see kSeedTiles)
    const uint32_t* deny;   // filtered-out inner ids as a bit mask, or null
};

// Cold start.  A wave that begins without a bound would have to sort its first tiles just to learn a
// threshold.  Instead every such wave publishes the smallest distance of its first tile into slot
// (global wave index mod k) of its query's seed row; waves own disjoint codes, so once all k slots are
// filled their maximum is a distance that k different codes reach -- a valid bound, usually far tighter
// than anything one wave could find alone.  A cold wave re-reads the row after each of its first
// kSeedTiles tiles; the host enables seeding only when there are at least 2k waves per query.
constexpr uint32_t kSeedTiles = 6;

template <int KIND, int METRIC, int T, bool SEED>
__global__ void __launch_bounds__(256)
flat_scan_kernel(ScanArgs a, FlatArgs f) {
    extern __shared__ uint64_t lds[];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nwaves = blockDim.x >> 6;
    const uint32_t S = f.S, k = f.k;
    uint64_t* sel = lds + static_cast<size_t>(wave) * T * S;

    uint32_t qidx[T];
    uint32_t thr[T];   // a candidate passes when its ordered distance is below thr
    uint32_t cnt[T];
    uint32_t cold[T];  // tiles after which this wave still looks at the seed row
    bool live[T];      // a real query that this launch serves
    bool any_live = false;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        qidx[t] = blockIdx.x * T + t;
        cnt[t] = 0;
        live[t] = qidx[t] < f.nq && (f.gate == nullptr || as_const(f.gate)[qidx[t]] != 0);
        any_live = any_live || live[t];
        uint32_t bs = live[t] ? __builtin_amdgcn_readfirstlane(__atomic_load_n(&f.bound[qidx[t]], __ATOMIC_RELAXED))
                              : 0xFFFFFFFFU;
        thr[t] = !live[t] ? 0U : bs == 0xFFFFFFFFU ? bs : bs + 1;
        cold[t] = SEED && live[t] && bs == 0xFFFFFFFFU ? kSeedTiles : 0;
    }
    if (!any_live) {
        return;
    }
    for (uint32_t i = lane; i < T * S; i += kWave) {
        sel[i] = kInfKey;
    }
    wave_lds_fence();
    const uint32_t seed_slot = (blockIdx.y * nwaves + wave) % k;

    const uint64_t tile_begin = f.tile0 + static_cast<uint64_t>(blockIdx.y) * f.tiles_per_chunk;
    uint64_t tile_end = tile_begin + f.tiles_per_chunk;
    if (tile_end > f.tile_end) {
        tile_end = f.tile_end;
    }
    // Software pipeline over granule groups: the loads of group g+1 (possibly of the next tile) are
    // issued before group g is consumed, so every wave keeps GROUP KiB in flight.  Two register buffers
    // alternate; the loop body is written out twice so that both are addressed statically.
    const QueryRows<T> qrows = query_rows<T>(a, qidx);
    constexpr int GROUP = GroupOf<T>::value;
    // RaBitQ codes have G = dim / 128 granules, often no multiple of the group (768 dimensions: 6).
    constexpr bool OVERLAP = KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32;
    TileStream<GROUP, OVERLAP> cur{a.tiles, lane, tile_begin + wave, tile_end, nwaves, 0, a.G};
    TileStream<GROUP, OVERLAP> nxt = cur;
    uint4 buf_a[GROUP], buf_b[GROUP];
    if (cur.valid()) {
        cur.load(buf_a, cur.tile);
    }
    Acc<KIND, T> acc;
    acc_reset(acc);

    const uint32_t pend = selector_base(S, k);  // where a selector's pending keys start
    // Sorts selector t and folds its k-th key and the shared bound into thr[t].
    auto flush = [&](int t) __attribute__((always_inline)) {
        uint64_t* keys = sel + t * S;
        uint64_t th = selector_flush(keys, S, k, cnt[t], lane);
        cnt[t] = 0;
        cold[t] = 0;
        uint32_t tl = static_cast<uint32_t>(th >> 32);  // 0xFFFFFFFF while fewer than k seen
        uint32_t bs = 0xFFFFFFFFU;
        if (live[t]) {
            bs = lower_shared(&f.bound[qidx[t]], tl, lane);  // tl = 0xFFFFFFFF lowers nothing
        }
        uint32_t tb = bs == 0xFFFFFFFFU ? bs : bs + 1;
        thr[t] = tl < tb ? tl : tb;
    };

    // What a cold wave reads of its queries' seed rows (largest entry over this lane's share): fetched when a tile
    // begins, looked at when its distances are done, so that the read waits under the tile's arithmetic.
    uint32_t seed_seen[T];
    auto consume = [&](const uint4(&regs)[GROUP]) __attribute__((always_inline)) {
        const uint32_t first = cur.first();
        if (SEED && cur.j0 == 0) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                seed_seen[t] = 0;
                if (cold[t] != 0) {
                    const uint32_t* row = f.seed + static_cast<uint64_t>(qidx[t]) * k;
                    for (uint32_t i = lane; i < k; i += kWave) {
                        const uint32_t v = __atomic_load_n(&row[i], __ATOMIC_RELAXED);
                        seed_seen[t] = v > seed_seen[t] ? v : seed_seen[t];
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const uint32_t g = first + u;
            if (g >= cur.j0 && g < a.G) {
                accumulate_granule<KIND, METRIC, T>(a, qrows, g, regs[u], acc);
            }
        }
        if (cur.j0 + GROUP < a.G) {
            return;
        }
        const uint64_t id = cur.tile * kWave + lane;
        float d[T];
        finish_distances<KIND, METRIC, T>(a, qidx, id, acc, d);
        acc_reset(acc);
        const bool valid = id < f.n && !denied(f.deny, id);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            // Inner ids grow along the scan, so "ordered distance < thr" is exactly the (distance, id)
            // order against the wave's own k-th key, and "<= bound" against the shared bound.
            uint32_t od = float_to_ordered(d[t]);
            if (SEED && cold[t] != 0) {
                uint32_t* row = f.seed + static_cast<uint64_t>(qidx[t]) * k;
                if (cold[t] == kSeedTiles) {
                    // This wave's entry (its own first look at the row came before it, the next one will see it).
                    uint32_t m = wave_min_u32(valid ? od : 0xFFFFFFFFU);
                    lower_shared(&row[seed_slot], m, lane);
                }
                --cold[t];
                const uint32_t mx = wave_max_u32(seed_seen[t]);
                if (mx != 0xFFFFFFFFU) {
                    // Every slot filled: k different codes reach mx.
                    cold[t] = 0;
                    const uint32_t b = lower_shared(&f.bound[qidx[t]], mx, lane);
                    thr[t] = b + 1 < thr[t] ? b + 1 : thr[t];
                }
            }
            bool pass = valid && od < thr[t];
            uint64_t mask = __ballot(pass);
            if (mask != 0) {
                uint32_t np = __popcll(mask);
                if (pend + cnt[t] + np > S) {
                    flush(t);
                }
                if (pass) {
                    sel[t * S + pend + cnt[t] + mask_rank(mask)] = (static_cast<uint64_t>(od) << 32) | static_cast<uint32_t>(id);
                }
                cnt[t] += np;
            }
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

    const uint32_t slot = f.slot0 + blockIdx.y * nwaves + wave;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (!live[t]) {
            continue;
        }
        // Whatever lies above the shared bound is beaten by k candidates of other waves.  What remains is
        // usually less than k keys, which go out as they are; only a wave left with more sorts once more.
        uint64_t* keys = sel + t * S;
        wave_lds_fence();
        uint32_t bs = __builtin_amdgcn_readfirstlane(__atomic_load_n(&f.bound[qidx[t]], __ATOMIC_RELAXED));
        uint32_t total = pend + cnt[t];
        uint32_t admitted = selector_count_admitted(keys, total, bs, lane);
        if (admitted > k) {
            uint64_t th = selector_flush(keys, S, k, cnt[t], lane);
            bs = lower_shared(&f.bound[qidx[t]], static_cast<uint32_t>(th >> 32), lane);
            total = k;
            admitted = selector_count_admitted(keys, total, bs, lane);
        }
        const uint64_t list = static_cast<uint64_t>(qidx[t]) * f.nslots + slot;
        if (lane == 0) {
            f.partial_cnt[list] = admitted;
        }
        if (admitted != 0) {
            selector_copy_admitted(keys, total, bs, f.partial + list * k, lane);
        }
    }
}

// Block-wide selection: the k-th smallest of keys[0, n) (all different), found by an 8-bit radix descent
// with LDS histograms; kInfKey when n < k.  Every thread of the workgroup calls it and gets the same value.
// Bytes that all keys share are skipped (the leading bytes of distances from one neighbourhood are equal, and
// a histogram with one occupied bin is 4096 atomics on one address); the descent stops as soon as the wanted
// key is alone in its bin.
struct SelectScratch {
    uint32_t hist[256];
    uint32_t bin;
    uint32_t before;
    uint32_t count;
    unsigned long long lo, hi, found;
};

__device__ inline uint64_t
block_kth_smallest(const uint64_t* keys, uint32_t n, uint32_t k, SelectScratch& sc) {
    if (n < k) {
        return kInfKey;
    }
    if (threadIdx.x == 0) {
        sc.lo = ~0ULL;
        sc.hi = 0ULL;
    }
    __syncthreads();
    {
        unsigned long long lo = ~0ULL, hi = 0ULL;
        for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
            unsigned long long key = keys[i];
            lo = key < lo ? key : lo;
            hi = key > hi ? key : hi;
        }
        for (int off = 32; off > 0; off >>= 1) {
            unsigned long long ol = __shfl_xor(lo, off), oh = __shfl_xor(hi, off);
            lo = ol < lo ? ol : lo;
            hi = oh > hi ? oh : hi;
        }
        if ((threadIdx.x & (kWave - 1)) == 0) {
            atomicMin(&sc.lo, lo);
            atomicMax(&sc.hi, hi);
        }
    }
    __syncthreads();
    const uint64_t spread = sc.lo ^ sc.hi;
    uint64_t prefix = 0;
    uint32_t want = k;  // rank of the wanted key among those that share the prefix
    for (int shift = 56; shift >= 0; shift -= 8) {
        if ((spread >> shift) == 0) {
            prefix |= sc.lo & (0xFFULL << shift);  // every key has this byte
            continue;
        }
        const uint64_t hi_mask = shift == 56 ? 0ULL : ~0ULL << (shift + 8);
        for (uint32_t i = threadIdx.x; i < 256; i += blockDim.x) {
            sc.hist[i] = 0;
        }
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
            uint64_t key = keys[i];
            if (((key ^ prefix) & hi_mask) == 0) {
                atomicAdd(&sc.hist[(key >> shift) & 255U], 1U);
            }
        }
        __syncthreads();
        if (threadIdx.x < kWave) {
            const uint32_t lane = threadIdx.x;
            uint32_t h[4] = {sc.hist[4 * lane], sc.hist[4 * lane + 1], sc.hist[4 * lane + 2], sc.hist[4 * lane + 3]};
            uint32_t sum = h[0] + h[1] + h[2] + h[3];
            uint32_t incl = sum;
            for (int off = 1; off < kWave; off <<= 1) {
                uint32_t o = __shfl_up(incl, off);
                if (static_cast<int>(lane) >= off) {
                    incl += o;
                }
            }
            uint32_t before = incl - sum;
            if (before < want && want <= incl) {
                uint32_t b = 0;
                while (before + h[b] < want) {
                    before += h[b];
                    ++b;
                }
                sc.bin = 4 * lane + b;
                sc.before = before;
                sc.count = h[b];
            }
        }
        __syncthreads();
        prefix |= static_cast<uint64_t>(sc.bin) << shift;
        want -= sc.before;
        const bool alone = sc.count == 1;
        __syncthreads();
        if (alone) {
            // One key left under this prefix: it is the answer.
            const uint64_t known = ~0ULL << shift;
            for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
                uint64_t key = keys[i];
                if (((key ^ prefix) & known) == 0) {
                    sc.found = key;
                }
            }
            __syncthreads();
            return sc.found;
        }
    }
    return prefix;
}

// Ascending bitonic sort of keys[0, P) (P a power of two) by the whole workgroup.
__device__ inline void
block_bitonic_sort(uint64_t* keys, uint32_t P) {
    for (uint32_t size = 2; size <= P; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t i = threadIdx.x; i < (P >> 1); i += blockDim.x) {
                uint32_t pos = 2 * i - (i & (stride - 1));
                uint64_t a = keys[pos];
                uint64_t b = keys[pos + stride];
                bool up = (pos & size) == 0;
                if ((a > b) == up) {
                    keys[pos] = b;
                    keys[pos + stride] = a;
                }
            }
            __syncthreads();
        }
    }
}

// One workgroup per query: the k best keys over its counted partial lists, written as ids / distances
// (ascending).  All threads first keep what the final shared bound admits (at least k keys when k exist) in
// an LDS pool; a radix selection finds the k-th smallest of the pool, the keys up to it are compacted and
// sorted.  When the pool overflows (long runs of nearly equal distances), the k-th smallest of what did fit
// -- an upper bound of the k-th smallest of all -- becomes the admission key of another round.
constexpr uint32_t kPoolKeys = 4096;       // few queries per call: every wave started without a bound
constexpr uint32_t kPoolKeysBatch = 2048;  // batches: the bound is known, and twice the workgroups fit a compute unit

__global__ void __launch_bounds__(1024)
merge_partials_kernel(const uint64_t* partial, const uint32_t* partial_cnt, const uint32_t* bound, uint32_t nslots,
                      uint32_t stride, uint32_t k, uint32_t S, uint32_t pool_keys, uint32_t* ids, float* dists) {
    extern __shared__ uint64_t lds[];  // S output keys, then the pool
    __shared__ uint32_t npool;
    __shared__ uint32_t nout;
    __shared__ SelectScratch scratch;
    constexpr uint32_t kLongLists = 128;
    __shared__ uint32_t nlong;
    __shared__ uint32_t long_slot[kLongLists];
    uint64_t* pool = lds + S;
    const uint64_t q = blockIdx.x;
    const uint32_t* cnts = partial_cnt + q * stride;  // the first nslots of the query's `stride` lists
    const uint64_t* src = partial + q * stride * k;
    uint64_t admit = (static_cast<uint64_t>(as_const(bound)[q]) << 32) | 0xFFFFFFFFULL;
    uint32_t sort_room = 2;  // keys the closing sort takes: the power of two from k on
    while (sort_room < k) {
        sort_room <<= 1;
    }
    // Finitely many rounds: every round that overflows lowers `admit` below at least one pooled key.
    for (;;) {
        if (threadIdx.x == 0) {
            npool = 0;
            nout = 0;
            nlong = 0;
        }
        __syncthreads();
        if (nslots * 4 <= blockDim.x) {
            // Few lists (the levels of a pre-selected batch): a wave per list, a lane per key.
            const uint32_t lane = threadIdx.x & (kWave - 1);
            for (uint32_t slot = threadIdx.x / kWave; slot < nslots; slot += blockDim.x / kWave) {
                const uint32_t c = cnts[slot];
                const uint64_t* list = src + static_cast<uint64_t>(slot) * k;
                for (uint32_t i0 = 0; i0 < c; i0 += kWave) {
                    const uint32_t i = i0 + lane;
                    const uint64_t key = i < c ? list[i] : kInfKey;
                    const bool keep = i < c && key <= admit;
                    const uint64_t votes = __ballot(keep);
                    if (votes == 0) {
                        continue;
                    }
                    uint32_t base = 0;
                    if (lane == 0) {
                        base = atomicAdd(&npool, static_cast<uint32_t>(__popcll(votes)));
                    }
                    base = __shfl(base, 0);
                    const uint32_t pos = base + static_cast<uint32_t>(__popcll(votes & ((1ULL << lane) - 1)));
                    if (keep && pos < pool_keys) {
                        pool[pos] = key;
                    }
                }
            }
        } else {
            // A thread per list: most lists are empty or nearly so once the bound is known.  The few long ones (the
            // lists of a query's nearest bucket hold up to k keys each) are noted and read a wave per list afterwards:
            // one thread walking such a list would outlast the whole workgroup.
            auto pool_key = [&](uint64_t key) {
                uint32_t pos = atomicAdd(&npool, 1U);
                if (pos < pool_keys) {
                    pool[pos] = key;
                }
            };
            for (uint32_t slot = threadIdx.x; slot < nslots; slot += blockDim.x) {
                const uint32_t c = cnts[slot];
                if (c > 4) {
                    const uint32_t at = atomicAdd(&nlong, 1U);
                    if (at < kLongLists) {
                        long_slot[at] = slot;
                        continue;
                    }
                }
                const uint64_t* list = src + static_cast<uint64_t>(slot) * k;
                // Four loads in flight at a time: the pool's atomics would otherwise serialise them.
                for (uint32_t i = 0; i < c; i += 4) {
                    uint64_t key[4];
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j) {
                        key[j] = i + j < c ? list[i + j] : kInfKey;
                    }
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j) {
                        if (i + j < c && key[j] <= admit) {
                            pool_key(key[j]);
                        }
                    }
                }
            }
            __syncthreads();
            const uint32_t lane = threadIdx.x & (kWave - 1);
            const uint32_t nl = nlong < kLongLists ? nlong : kLongLists;
            for (uint32_t w = threadIdx.x / kWave; w < nl; w += blockDim.x / kWave) {
                const uint32_t slot = long_slot[w];
                const uint32_t c = cnts[slot];
                const uint64_t* list = src + static_cast<uint64_t>(slot) * k;
                for (uint32_t i0 = 0; i0 < c; i0 += kWave) {
                    const uint32_t i = i0 + lane;
                    const uint64_t key = i < c ? list[i] : kInfKey;
                    const bool keep = i < c && key <= admit;
                    const uint64_t votes = __ballot(keep);
                    if (votes == 0) {
                        continue;
                    }
                    uint32_t base = 0;
                    if (lane == 0) {
                        base = atomicAdd(&npool, static_cast<uint32_t>(__popcll(votes)));
                    }
                    base = __shfl(base, 0);
                    const uint32_t pos = base + static_cast<uint32_t>(__popcll(votes & ((1ULL << lane) - 1)));
                    if (keep && pos < pool_keys) {
                        pool[pos] = key;
                    }
                }
            }
        }
        __syncthreads();
        const uint32_t total = npool;
        const uint32_t n = total < pool_keys ? total : pool_keys;
        if (total <= sort_room) {
            // The usual case once the bound is tight: hardly more than k keys are admitted, and the sort that follows
            // orders them all without a selection first.
            for (uint32_t i = threadIdx.x; i < total; i += blockDim.x) {
                lds[i] = pool[i];
            }
            if (threadIdx.x == 0) {
                nout = total;
            }
            break;
        }
        const uint64_t kth = block_kth_smallest(pool, n, k, scratch);
        if (total <= pool_keys) {
            // The k smallest (all of them when fewer than k) go to the front of the output area: what lies below the
            // k-th first, then as many copies of the k-th key as still fit (a list probed twice by one query brings
            // every key twice).
            for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
                uint64_t key = pool[i];
                if (key < kth) {
                    lds[atomicAdd(&nout, 1U)] = key;
                }
            }
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
                if (pool[i] == kth) {
                    const uint32_t pos = atomicAdd(&nout, 1U);
                    if (pos < sort_room) {
                        lds[pos] = kth;
                    }
                }
            }
            __syncthreads();
            if (threadIdx.x == 0 && nout > sort_room) {
                nout = sort_room;
            }
            break;
        }
        admit = kth;
        __syncthreads();
    }
    __syncthreads();
    uint32_t P = 2;
    while (P < k) {
        P <<= 1;
    }
    for (uint32_t i = nout + threadIdx.x; i < P; i += blockDim.x) {
        lds[i] = kInfKey;
    }
    __syncthreads();
    block_bitonic_sort(lds, P);
    for (uint32_t i = threadIdx.x; i < k; i += blockDim.x) {
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

// The same for a handful of short lists (the levels of a pre-selected batch with a small k): one wave per query, the
// admitted keys sorted in LDS.  Every list holds at most k keys, so nslots * k keys of room never overflow.
constexpr uint32_t kSmallMergeKeys = 512;

__global__ void __launch_bounds__(64)
merge_small_kernel(const uint64_t* partial, const uint32_t* partial_cnt, const uint32_t* bound, uint32_t nslots,
                   uint32_t stride, uint32_t k, uint32_t* ids, float* dists) {
    __shared__ uint64_t pool[kSmallMergeKeys];
    const uint32_t lane = threadIdx.x;
    const uint64_t q = blockIdx.x;
    const uint32_t* cnts = partial_cnt + q * stride;
    const uint64_t* src = partial + q * stride * k;
    const uint64_t admit = (static_cast<uint64_t>(as_const(bound)[q]) << 32) | 0xFFFFFFFFULL;
    const uint32_t mine = lane < nslots ? cnts[lane] : 0U;  // nslots <= 64
    uint32_t fill = 0;
    uint64_t lists = __ballot(mine != 0);
    while (lists != 0) {
        const uint32_t slot = static_cast<uint32_t>(__builtin_ctzll(lists));
        lists &= lists - 1;
        const uint32_t c = __shfl(mine, static_cast<int>(slot));
        const uint64_t* list = src + static_cast<uint64_t>(slot) * k;
        for (uint32_t i0 = 0; i0 < c; i0 += kWave) {
            const uint32_t i = i0 + lane;
            const uint64_t key = i < c ? list[i] : kInfKey;
            const bool keep = i < c && key <= admit;
            const uint64_t votes = __ballot(keep);
            if (keep) {
                pool[fill + static_cast<uint32_t>(__popcll(votes & ((1ULL << lane) - 1)))] = key;
            }
            fill += static_cast<uint32_t>(__popcll(votes));
        }
    }
    uint32_t P = 2;
    while (P < fill || P < k) {
        P <<= 1;
    }
    P = P > kSmallMergeKeys ? kSmallMergeKeys : P;  // k <= nslots * k <= kSmallMergeKeys, a power of two
    for (uint32_t i = fill + lane; i < P; i += kWave) {
        pool[i] = kInfKey;
    }
    wave_lds_fence();
    for (uint32_t size = 2; size <= P; size <<= 1) {
        for (uint32_t step = size >> 1; step > 0; step >>= 1) {
            for (uint32_t t = lane; t < P / 2; t += kWave) {
                const uint32_t pos = 2 * t - (t & (step - 1));
                const uint64_t x = pool[pos], y = pool[pos + step];
                const bool up = (pos & size) == 0;
                if ((x > y) == up) {
                    pool[pos] = y;
                    pool[pos + step] = x;
                }
            }
            wave_lds_fence();
        }
    }
    for (uint32_t i = lane; i < k; i += kWave) {
        const uint64_t key = pool[i];
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
int
launch_merge_partials(const uint64_t* partial, const uint32_t* partial_cnt, const uint32_t* bound, uint32_t nslots,
                      uint32_t stride, uint32_t k, uint32_t S, uint64_t nq, uint32_t* ids, float* dists,
                      hipStream_t st) {
    if (nslots <= kWave && static_cast<uint64_t>(nslots) * k <= kSmallMergeKeys && nq > 256) {
        hipLaunchKernelGGL(merge_small_kernel, dim3(static_cast<uint32_t>(nq)), dim3(kWave), 0, st, partial, partial_cnt,
                           bound, nslots, stride, k, ids, dists);
        VA_HIP(hipGetLastError());
        return 0;
    }
    // Few queries: many candidates each (every wave starts without a bound), so give each merge more threads.
    const uint32_t threads = nq <= 256 ? 1024 : 256;
    const uint32_t pool_keys = nq <= 256 ? kPoolKeys : kPoolKeysBatch;
    hipLaunchKernelGGL(merge_partials_kernel, dim3(static_cast<uint32_t>(nq)), dim3(threads), (S + pool_keys) * 8, st,
                       partial, partial_cnt, bound, nslots, stride, k, S, pool_keys, ids, dists);
    VA_HIP(hipGetLastError());
    return 0;
}

static int g_tile_override = 0;
static int g_chunk_override = 0;
// A store's own setting (vsag_amd_store_set_scan_tuning) goes before the process-wide one.
static int tile_override(const vsag_amd_store* s) { return s->tile_override >= 0 ? s->tile_override : g_tile_override; }
static int chunk_override(const vsag_amd_store* s) { return s->chunk_override >= 0 ? s->chunk_override : g_chunk_override; }
static thread_local int tl_last_tile = 0;
static thread_local uint64_t tl_last_passes = 0;
static thread_local uint64_t tl_last_bytes = 0;

// Queries per wave.  More queries per pass means fewer passes over the codes but more scalar registers;
// these are the largest tiles that still compile without spilling.
static int
default_query_tile(const vsag_amd_store* s) {
    switch (s->kind) {
        case VSAG_AMD_KIND_SQ8:
        case VSAG_AMD_KIND_SQ4:
            return 4;
        case VSAG_AMD_KIND_RABITQ:
            return 2;
        default:
            return 4;
    }
}

struct ScanPlan {
    int T;
    uint32_t S;
    uint32_t waves;
    uint64_t groups;     // grid x
    uint64_t nq_pad;
    uint64_t chunks;     // grid y
    uint64_t tiles_per_chunk;
    size_t lds_bytes;
    QueryLayout ql;
    size_t qcode_bytes;  // staging for encoded queries (uniform kinds, rabitq)
    bool seeded;         // cold waves learn a bound from each other's first tiles (kSeedTiles)
};

static void
make_plan(const vsag_amd_store* s, uint64_t nq, uint32_t k, uint64_t ntiles, ScanPlan* p) {
    p->S = selector_slots(k);
    int T = tile_override(s) > 0 ? tile_override(s) : default_query_tile(s);
    if (tile_override(s) <= 0 && s->kind == VSAG_AMD_KIND_FP32 && ntiles >= 1024) {
        // 512 bytes per code and pass: on a long scan the passes are what costs (100k x 128: a quarter faster than 4);
        // short scans (centroid routing, the exact prefix of a pre-selected batch) live on their selectors instead.
        T = 8;
    }
    if (tile_override(s) <= 0 && T > 2 && ntiles <= 32 && nq >= 2048) {
        // A few tiles under thousands of queries (the exact prefix of a pre-selected batch): the scan lives on its
        // selectors, and two queries per wave mean twice the waves to overlap each other's flushes (1M x 128 sq8 codes,
        // 10 000 queries: the prefix launch 188 -> 157 us).
        T = 2;
    }
    while (T > 1 && static_cast<uint64_t>(T) > nq) {
        T >>= 1;
    }
    const size_t lds_budget = 65536;
    while (T > 1 && static_cast<size_t>(T) * p->S * 8 > lds_budget) {
        T >>= 1;
    }
    uint32_t waves = kMaxWaves;
    while (waves > 1 && static_cast<size_t>(waves) * T * p->S * 8 > lds_budget) {
        waves >>= 1;
    }
    // A short scan under many queries (centroid routing, the exact prefix of a pre-selected batch): every wave of a
    // workgroup keeps selectors of its own for the same queries, so with a few tiles per wave the selecting outweighs
    // the scanning.  Fewer waves then, as long as the grid still holds two waves per SIMD of the machine.
    const uint64_t groups_all = div_up(nq, static_cast<uint64_t>(T));
    while (waves > 1 && ntiles / waves < 32 && groups_all * (waves / 2) >= static_cast<uint64_t>(device_cu_count()) * 8) {
        waves >>= 1;
    }
    p->T = T;
    p->waves = waves;
    p->lds_bytes = static_cast<size_t>(waves) * T * p->S * 8;
    p->groups = div_up(nq, static_cast<uint64_t>(T));
    p->nq_pad = p->groups * T;
    uint64_t chunks;
    if (chunk_override(s) > 0) {
        chunks = chunk_override(s);
    } else {
        // Workgroups in the grid: about 64 per query group, but at least two per compute unit (few queries:
        // every wave still has a long run of tiles behind its cold start) and at most eight rounds of
        // workgroups over the machine (eight fit a compute unit).
        uint64_t want = 64 * p->groups;
        const uint64_t lo = static_cast<uint64_t>(device_cu_count()) * 2, hi = static_cast<uint64_t>(device_cu_count()) * 64;
        want = want < lo ? lo : want > hi ? hi : want;
        chunks = div_up(want, p->groups);
    }
    // At least 16 tiles per wave -- fewer (down to one) when the store is so small that this would leave
    // most of the machine without a workgroup (centroid routing, small indexes).
    uint64_t tiles_min = 16;
    while (tiles_min > 1 && p->groups * (ntiles / (tiles_min * waves)) < static_cast<uint64_t>(device_cu_count())) {
        tiles_min >>= 1;
    }
    uint64_t max_chunks = ntiles / (tiles_min * waves);
    if (max_chunks < 1) {
        max_chunks = 1;
    }
    if (chunks > max_chunks) {
        chunks = max_chunks;
    }
    if (chunks > 65535) {
        chunks = 65535;
    }
    p->tiles_per_chunk = div_up(ntiles > 0 ? ntiles : 1, chunks);
    p->chunks = div_up(ntiles > 0 ? ntiles : 1, p->tiles_per_chunk);
    // Seeding pays when a query's waves all start cold together, i.e. when the whole grid is resident at once.
    p->seeded = p->chunks * waves >= 2ull * k && k <= 256 && p->groups * p->chunks * waves <= 8192;
    p->ql = query_layout(s);
    p->qcode_bytes = query_staging_bytes(s, nq);
}

// A call is served either by one streaming launch over all tiles, or -- large batches on fp32 / sq8 stores
// (prefilter.hip) -- by a streaming launch over a prefix, the matrix-core prefilter with exact rescoring over the
// rest, and a streaming launch over the rest for the queries whose candidates overflowed.
struct CallPlan {
    ScanPlan all;
    bool contraction = false;
    ScanPlan prefix, rest;
    uint64_t prefix_tiles = 0;
    // The tiles behind the prefix are pre-selected level by level, each level against the k-th distance of
    // everything before it: level l covers tiles [level_begin[l], level_begin[l + 1]).
    static constexpr int kMaxLevels = 8;
    int levels = 0;
    uint64_t level_begin[kMaxLevels + 1] = {};
    bool int8 = false;         // the int8 matrix cores pre-select (sq8, at most 128 dimensions)
    bool rb = false;           // RaBitQ store: 1-bit codes x 4-bit queries on the int8 matrix cores
    size_t h16_scratch = 0;    // sq8 beyond 128 dimensions: bytes of the fp16 query planes (0: the fp32 matrix cores)
    uint32_t cap = 0;          // candidates per query and level
    uint32_t sub_lists[kMaxLevels] = {};  // int8: private candidate lists per query ...
    uint32_t sub_cap[kMaxLevels] = {};    // ... of this many slots
    uint32_t max_lists = 0;    // the largest sub_lists
    size_t rb_scratch = 0;     // rb: bytes of the expanded queries and per-query factors
    uint32_t nslots = 0;       // partial lists per query
    bool any_seeded = false;
    // Many queries against a small fp32 store (the routing of an ivf search): a table of approximate distances from the
    // fp32 matrix cores, then per query the exact distances of the few codes that can be among the k best.
    bool table = false;
    uint64_t table_ld = 0;     // floats per row of the table
    // One query against a large store (scan_one.hip): a pass that writes every distance and a minimum per run of
    // tiles, then a one-workgroup selection.
    bool one = false;
    uint32_t one_runs = 0;
    uint64_t one_tiles = 0;
};

// -1 never, 0 when it pays, 1 whenever the store supports it, 2 like 1 but on the fp32 matrix cores only
static int g_prefilter_mode = 0;
// A store's own setting (vsag_amd_store_set_scan_contraction) goes before the process-wide one.
static int prefilter_mode(const vsag_amd_store* s) { return s->contraction_mode >= -1 ? s->contraction_mode : g_prefilter_mode; }

bool one_query_supports(const vsag_amd_store* s, uint64_t nq, uint32_t k);
uint32_t one_query_run_tiles(const vsag_amd_store* s);
int launch_one_query(const vsag_amd_store* s, const ScanArgs& a, uint32_t k, const vsag_amd_search_options_t* options,
                     uint32_t* dist, uint64_t* mins, uint32_t* ids_dev, float* dists_dev, hipStream_t st);
bool prefilter_supports(const vsag_amd_store* s);
int launch_prefilter(const vsag_amd_store* s, const ScanArgs& a, uint64_t nq, uint32_t k, uint32_t S, uint64_t tile_begin,
                     uint64_t tile_end, uint32_t* bound, float* tau, uint32_t* cand, uint32_t* cand_cnt, uint32_t cap,
                     uint64_t* partial, uint32_t* partial_cnt, uint32_t nslots, uint32_t first_slot, uint32_t out_slot,
                     uint32_t* gate, uint8_t* q8, float* q8_u, uint32_t sub_lists, uint32_t sub_cap,
                     const float* merged_dists, hipStream_t st);
bool prefilter_i8_supports(const vsag_amd_store* s);
size_t prefilter_i8_query_bytes(uint64_t nq);
size_t prefilter_i8_scalar_floats(uint64_t nq);
uint32_t prefilter_i8_sub_lists(uint64_t nq, uint64_t span);
bool prefilter_rb_supports(const vsag_amd_store* s);
size_t prefilter_rb_scratch_bytes(const vsag_amd_store* s, uint64_t nq);
bool prefilter_h16_supports(const vsag_amd_store* s);
size_t prefilter_h16_scratch_bytes(const vsag_amd_store* s, uint64_t nq);
uint32_t prefilter_rb_sub_lists(uint64_t nq, uint64_t span);

// Whether a call goes through the table of approximate distances (see CallPlan::table).
constexpr uint64_t kTableMinCodes = 1024, kTableMaxCodes = 8192;
constexpr uint32_t kTableMaxK = 256;
static bool
small_store_table(const vsag_amd_store* s, uint64_t nq, uint32_t k) {
    return s->kind == VSAG_AMD_KIND_FP32 && s->nlist == 0 && prefilter_mode(s) == 0 && nq >= 1024 && k <= kTableMaxK &&
           s->n >= kTableMinCodes && s->ntiles * kWave <= kTableMaxCodes && nq * (s->ntiles * kWave) * 4 <= (2ull << 30);
}

static void
make_call_plan(const vsag_amd_store* s, uint64_t nq, uint32_t k, CallPlan* c) {
    make_plan(s, nq, k, s->ntiles, &c->all);
    c->nslots = static_cast<uint32_t>(c->all.chunks * c->all.waves);
    c->any_seeded = c->all.seeded;
    c->contraction = false;
    c->table = small_store_table(s, nq, k);
    c->table_ld = c->table ? round_up(s->ntiles * kWave, 64) : 0;
    if (c->table) {
        return;
    }
    // (an explicit query tile asks for the streaming kernel)
    c->one = tile_override(s) <= 0 && one_query_supports(s, nq, k);
    c->one_runs = c->one ? static_cast<uint32_t>(div_up(s->ntiles, static_cast<uint64_t>(one_query_run_tiles(s)))) : 0;
    c->one_tiles = c->one ? s->ntiles : 0;
    if (prefilter_mode(s) < 0 || !prefilter_supports(s)) {
        return;
    }
    const bool forced = prefilter_mode(s) > 0;
    const bool rb = prefilter_rb_supports(s);
    if (!forced && (nq < 512 || k > (rb ? 256U : 128U) || s->ntiles < 1024)) {
        return;
    }
    // Candidate buffers: at most 2 GiB in all, 1024 to 4096 candidates per query (RaBitQ stores are searched with
    // hundreds of candidates for a later rerank: eight times as many).
    uint64_t cap = rb ? 32768 : 4096;
    while (cap > 1024 && nq * cap * 4 > (2ull << 30)) {
        cap /= 2;
    }
    if (nq * cap * 4 > (2ull << 30)) {
        return;
    }
    // A level behind b tiles admits about k * (its tiles / b) codes per query: with every boundary a factor r
    // behind the next one that is k * r, kept below an eighth of the buffer.  The prefix in front of the first
    // level is scanned exactly by the streaming kernel.
    // Every level also costs a merge of the lists so far, every admitted code an exact rescoring: with the hundreds
    // of candidates a RaBitQ search keeps, the rescoring of k * r codes per query and level outweighs the merges
    // unless r is small.
    uint64_t r = std::min<uint64_t>(16, std::max<uint64_t>(2, cap / (8ull * k)));
    if (rb) {
        r = std::min<uint64_t>(r, std::max<uint64_t>(3, 600 / k));
    }
    // The int8 matrix cores pass a tile forty times faster than the streaming kernel: there a short exact prefix and
    // one more level beat a long prefix.
    const bool i8 = prefilter_i8_supports(s) && !rb;
    if (i8) {
        // Every candidate costs the int8 kernel a detour out of its matrix-instruction stream and the rescoring a
        // gathered row, every level a handful of small launches: with levels a factor 6 apart the two meet
        // (1M codes, 10 000 queries: 2.86 ms per call against 2.98 ms at a factor 16 and 3.00 ms at a factor 4).
        r = std::min<uint64_t>(r, 6);
    }
    // (The fp16 pass of sq8 stores beyond 128 dimensions is ten times the streaming kernel: a short prefix there too.)
    // (Mode 2 asks for the fp32 matrix cores, which sq4 has no route for.)
    const bool h16 = !i8 && !rb && (prefilter_mode(s) != 2 || s->kind == VSAG_AMD_KIND_SQ4) && prefilter_h16_supports(s);
    const uint64_t min_prefix = forced ? 2 : (i8 || h16 ? std::max<uint64_t>(8, div_up(4ull * k, kWave)) : 64);
    uint64_t bounds[CallPlan::kMaxLevels + 1];
    int nb = 0;
    bounds[nb++] = s->ntiles;
    uint64_t cur = s->ntiles;
    while (nb <= CallPlan::kMaxLevels) {
        uint64_t next = std::max(min_prefix, div_up(cur, r));
        next += next & 1;
        if (nb > 1 && cur < std::min<uint64_t>(4, r / 2) * next) {
            break;  // too thin a level to be worth its launches
        }
        bounds[nb++] = next;
        cur = next;
        if (next == min_prefix) {
            break;
        }
    }
    const uint64_t prefix = bounds[nb - 1];
    if (nb < 2 || prefix > s->ntiles / (forced ? 2 : 4) || prefix >= s->ntiles) {
        return;
    }
    c->contraction = true;
    // Mode 2 asks for the fp32 matrix cores, which the uniform kinds have no route for.
    c->int8 = prefilter_i8_supports(s) && (prefilter_mode(s) != 2 || s->kind == VSAG_AMD_KIND_SQ8_UNIFORM ||
                                           s->kind == VSAG_AMD_KIND_SQ4_UNIFORM || s->kind == VSAG_AMD_KIND_SQ4);
    c->rb = rb;
    c->rb_scratch = rb ? prefilter_rb_scratch_bytes(s, nq) : 0;
    // (mode 2 keeps the fp32 matrix cores)
    c->h16_scratch = h16 && !c->int8 ? prefilter_h16_scratch_bytes(s, nq) : 0;
    c->prefix_tiles = prefix;
    c->cap = static_cast<uint32_t>(cap);
    c->levels = nb - 1;
    for (int l = 0; l <= c->levels; ++l) {
        c->level_begin[l] = bounds[nb - 1 - l];
    }
    c->max_lists = 0;
    if (c->rb) {
        for (int l = 0; l < c->levels; ++l) {
            c->sub_lists[l] = prefilter_rb_sub_lists(nq, c->level_begin[l + 1] - c->level_begin[l]);
            c->sub_cap[l] = std::max<uint32_t>(16, static_cast<uint32_t>(div_up(cap, static_cast<uint64_t>(c->sub_lists[l]))));
            c->sub_cap[l] = std::min<uint32_t>(c->sub_cap[l], 4096);  // what the rescoring gathers at a time
            c->cap = std::max(c->cap, c->sub_lists[l] * c->sub_cap[l]);
            c->max_lists = std::max(c->max_lists, c->sub_lists[l]);
        }
    }
    if (c->int8) {
        for (int l = 0; l < c->levels; ++l) {
            // The expected load of a list is an eighth of its share of the buffer; short lists get room for the
            // tail of that distribution.
            c->sub_lists[l] = prefilter_i8_sub_lists(nq, c->level_begin[l + 1] - c->level_begin[l]);
            c->sub_cap[l] = std::max<uint32_t>(16, static_cast<uint32_t>(div_up(cap, static_cast<uint64_t>(c->sub_lists[l]))));
            c->cap = std::max(c->cap, c->sub_lists[l] * c->sub_cap[l]);
            c->max_lists = std::max(c->max_lists, c->sub_lists[l]);
        }
    }
    make_plan(s, nq, k, prefix, &c->prefix);
    make_plan(s, nq, k, s->ntiles - prefix, &c->rest);
    uint32_t pf_slots = static_cast<uint32_t>(c->prefix.chunks * c->prefix.waves + c->levels + c->rest.chunks * c->rest.waves);
    c->nslots = std::max(c->nslots, pf_slots);
    c->any_seeded = c->any_seeded || c->prefix.seeded || c->rest.seeded;
}

struct ScanBuffers {
    uint32_t* qtab;
    float* qmeta;
    uint8_t* qcodes;
    uint32_t* bound;
    uint32_t* partial_cnt;
    uint64_t* partial;
    uint32_t* seed;  // null when no launch of the plan seeds
    // contraction only
    float* tau;
    uint32_t* cand_cnt;
    uint32_t* gate;
    uint32_t* cand;
    uint8_t* q8;   // int8 planes of the queries, null on the fp32 matrix cores
    float* q8_u;
    // table route only
    float* table;       // nq x table_ld approximate distances
    float* table_rows;  // the codes a row per code
    float* table_norms; // their squared norms, then (one word) the largest as float bits
    // one-query route only
    uint32_t* one_dist;  // an ordered distance per tile slot
    uint64_t* one_mins;  // the smallest key per run of tiles
};

static size_t
carve_scan(Carver& c, const CallPlan& cp, uint64_t nq, uint32_t k, ScanBuffers* b) {
    const ScanPlan& p = cp.all;
    b->qtab = c.take<uint32_t>(p.nq_pad * p.ql.qstride);
    b->qmeta = c.take<float>(p.nq_pad * p.ql.qmeta);
    b->qcodes = c.take<uint8_t>(p.qcode_bytes);
    b->bound = c.take<uint32_t>(nq);
    b->partial_cnt = c.take<uint32_t>(nq * cp.nslots);
    b->seed = c.take<uint32_t>(cp.any_seeded ? nq * k : 0);
    if (!cp.any_seeded) {
        b->seed = nullptr;
    }
    b->partial = c.take<uint64_t>(nq * cp.nslots * k);
    const uint64_t nq_pad8 = prefilter_i8_query_bytes(nq) / 256;  // whole workgroups of the int8 prefilter
    b->tau = c.take<float>(cp.contraction ? nq_pad8 : 0);
    b->q8_u = c.take<float>(cp.int8 ? prefilter_i8_scalar_floats(nq) : 0);
    b->q8 = c.take<uint8_t>(cp.int8 ? prefilter_i8_query_bytes(nq) : (cp.rb ? cp.rb_scratch : cp.h16_scratch));
    if (!cp.int8 && !cp.rb && cp.h16_scratch == 0) {
        b->q8 = nullptr;
    }
    b->cand_cnt = c.take<uint32_t>(cp.contraction ? nq * std::max<uint32_t>(1, cp.max_lists) : 0);
    b->gate = c.take<uint32_t>(cp.contraction ? nq : 0);
    b->cand = c.take<uint32_t>(cp.contraction ? nq * cp.cap : 0);
    b->table = c.take<float>(cp.table ? nq * cp.table_ld : 0);
    b->table_rows = c.take<float>(cp.table ? cp.table_ld * p.ql.qstride : 0);
    b->table_norms = c.take<float>(cp.table ? cp.table_ld + 64 : 0);
    b->one_mins = c.take<uint64_t>(cp.one ? cp.one_runs : 0);
    b->one_dist = c.take<uint32_t>(cp.one ? cp.one_tiles * kWave : 0);
    return c.used;
}

template <int KIND, int METRIC, int T>
static void
launch_flat_s(dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a, const FlatArgs& f) {
    if (f.seed != nullptr) {
        hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, T, true>), grid, block, lds, st, a, f);
    } else {
        hipLaunchKernelGGL((flat_scan_kernel<KIND, METRIC, T, false>), grid, block, lds, st, a, f);
    }
}

template <int KIND, int METRIC>
static void
launch_flat_t(int T, dim3 grid, dim3 block, size_t lds, hipStream_t st, const ScanArgs& a, const FlatArgs& f) {
    switch (T) {
        case 1:
            launch_flat_s<KIND, METRIC, 1>(grid, block, lds, st, a, f);
            break;
        case 2:
            launch_flat_s<KIND, METRIC, 2>(grid, block, lds, st, a, f);
            break;
        case 4:
            launch_flat_s<KIND, METRIC, 4>(grid, block, lds, st, a, f);
            break;
        default:
            launch_flat_s<KIND, METRIC, 8>(grid, block, lds, st, a, f);
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
    } else if (metric == VSAG_AMD_METRIC_COSINE && (KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32)) {
        launch_flat_t<KIND, VSAG_AMD_METRIC_COSINE>(T, grid, block, lds, st, a, f);
    } else {
        launch_flat_t<KIND, VSAG_AMD_METRIC_IP>(T, grid, block, lds, st, a, f);
    }
}

static int
launch_flat(const vsag_amd_store* s, const ScanPlan& p, const ScanArgs& a, const FlatArgs& f, hipStream_t st) {
    dim3 grid(static_cast<uint32_t>(p.groups), static_cast<uint32_t>(p.chunks));
    dim3 block(p.waves * kWave);
    size_t lds = p.lds_bytes;
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
        case VSAG_AMD_KIND_PQFS:
            launch_flat_m<VSAG_AMD_KIND_PQFS>(s->metric, p.T, grid, block, lds, st, a, f);
            break;
        case VSAG_AMD_KIND_RABITQ:
            if (s->query_bits == 32) {
                launch_flat_m<kKindRabitqF32>(s->metric, p.T, grid, block, lds, st, a, f);
            } else {
                launch_flat_m<VSAG_AMD_KIND_RABITQ>(s->metric, p.T, grid, block, lds, st, a, f);
            }
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

// ---- many queries against a small fp32 store: selection from a table of approximate distances ------------------
// (the routing of an ivf search over its centroids: 10 000 queries x 4096 centroids x 128 dimensions).  The streaming
// distance sum (q_d - c_d)^2 is a subtraction and an fma per dimension; on the vector ALU that alone is 0.27 ms here.
// The fp32 matrix cores deliver |c|^2 - 2 <q, c> (inner product: -<q, c>) for every pair in a third of that
// (kmeans.hip, launch_row_products), but rounded differently.  So the table only selects: with a_k the k-th smallest
// table value of a query and eps a bound on |table - streaming distance| (up to the query's own constant), every code
// among the k best by streaming distance has a table value of at most a_k + 2 eps; those few codes -- k and a
// handful -- get their streaming distance, and the k best of them are the result, bit for bit what the streaming
// scan returns.
int launch_row_products(const float* x, uint64_t nx, const float* c, uint32_t nc, uint32_t dim, const float* base, float alpha,
                        float* out, uint64_t ld, hipStream_t st);
int launch_row_sqnorms(const float* x, uint64_t nx, uint32_t dim, float* out, uint32_t* max_bits, hipStream_t st);

constexpr uint32_t kTablePool = 512;  // candidates a query may have before it is redone by a full scan

// rows[slot][4 j ...] = granule j of the code in `slot`: rows of `row_granules` granules like the rows of the query
// table (zero behind the code's own G granules, zero rows behind the last code).
__global__ void __launch_bounds__(256)
table_rows_kernel(const uint4* tiles, uint32_t G, uint32_t row_granules, uint64_t n, uint64_t slots, float* rows,
                  uint32_t* max_bits) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i == 0) {
        *max_bits = 0;
    }
    if (i >= slots * row_granules) {
        return;
    }
    const uint64_t slot = i / row_granules;
    const uint32_t j = static_cast<uint32_t>(i % row_granules);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (slot < n && j < G) {
        v = tiles[((slot / kWave) * G + j) * kWave + slot % kWave];
    }
    reinterpret_cast<uint4*>(rows)[slot * row_granules + j] = v;
}

// The exact scan of one query (row qi of the query table) by one wave: all keys at or below `limit`, the k best written
// out.  The pool takes kTablePool keys; when more lie at or below the limit, the k-th of what was pooled (an upper bound
// of the k-th of all that lies below at least kTablePool - k pooled keys) is the limit of another pass.
template <int METRIC>
__device__ inline void
table_redo(const ScanArgs& a, uint64_t n, uint64_t ntiles, uint32_t k, uint32_t qi, uint32_t* ids, float* dists,
           uint64_t limit, uint64_t* pool, uint32_t lane) {
    const uint32_t qidx[1] = {qi};
    const QueryRows<1> qrows = query_rows<1>(a, qidx);
    for (;;) {
        uint32_t count = 0;
        for (uint64_t tile = 0; tile < ntiles; ++tile) {
            Acc<VSAG_AMD_KIND_FP32, 1> acc;
            acc_reset(acc);
            for (uint32_t j = 0; j < a.G; ++j) {
                accumulate_granule<VSAG_AMD_KIND_FP32, METRIC, 1>(a, qrows, j, a.tiles[(tile * a.G + j) * kWave + lane], acc);
            }
            const uint64_t slot = tile * kWave + lane;
            float d[1];
            finish_distances<VSAG_AMD_KIND_FP32, METRIC, 1>(a, qidx, slot, acc, d);
            const uint64_t key = make_key(d[0], static_cast<uint32_t>(slot));
            const bool pass = slot < n && key <= limit;
            const uint64_t mask = __ballot(pass);
            const uint32_t at = count + mask_rank(mask);
            if (pass && at < kTablePool) {
                pool[at] = key;
            }
            count += static_cast<uint32_t>(__popcll(mask));
        }
        const uint32_t kept = count < kTablePool ? count : kTablePool;
        for (uint32_t i = kept + lane; i < kTablePool; i += kWave) {
            pool[i] = kInfKey;
        }
        wave_lds_fence();
        wave_bitonic_sort(pool, kTablePool, lane);
        if (count <= kTablePool) {
            break;
        }
        limit = wave_uniform_u64(pool[k - 1]);
        wave_lds_fence();
    }
    for (uint32_t i = lane; i < k; i += kWave) {
        const uint64_t key = pool[i];
        ids[i] = key == kInfKey ? VSAG_AMD_INVALID_ID : static_cast<uint32_t>(key);
        dists[i] = key == kInfKey ? __builtin_inff() : ordered_to_float(static_cast<uint32_t>(key >> 32));
    }
}

struct TableSelectArgs {
    const float* table;  // nq x ld
    uint64_t ld;
    uint64_t nq, n, ntiles;
    uint32_t k, dim;
    const uint32_t* max_norm_bits;  // the largest |c|^2
    uint32_t* ids;
    float* dists;
    const uint4* rows;      // the codes a row per code, row_granules granules each: a candidate's granules lie together
    uint32_t row_granules;  // there (eight cache lines for 128 dimensions against 32 in the tiles)
};

// One wave per query; NV table values per lane (NV * 64 >= the codes of the store).
template <int METRIC, int NV>
__global__ void __launch_bounds__(64)
table_select_kernel(ScanArgs a, TableSelectArgs p) {
    __shared__ uint64_t pool[kTablePool];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t cand[kTablePool];
    const uint32_t lane = threadIdx.x;
    const uint64_t q = blockIdx.x;
    const float* row = p.table + q * p.ld;
    float val[NV];
    bool odd = false;  // a value that is no number: the table cannot order this query
    float vmin = __builtin_inff(), vmax = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint64_t c = static_cast<uint64_t>(i) * kWave + lane;
        val[i] = c < p.n ? row[c] : __builtin_inff();
        odd = odd || val[i] != val[i];
        if (c < p.n) {
            vmin = fminf(vmin, val[i]);
            vmax = fmaxf(vmax, val[i]);
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        vmin = fminf(vmin, __shfl_xor(vmin, off));
        vmax = fmaxf(vmax, __shfl_xor(vmax, off));
    }
    // |table - streaming| <= eps: both sums run over dim terms in fp32, whatever their order.
    const uint32_t* qrow = a.qtab + q * a.qstride;
    float qn2 = 0.0F;
    for (uint32_t d = lane; d < a.qstride; d += kWave) {
        const float x = __uint_as_float(qrow[d]);
        qn2 = fmaf(x, x, qn2);
    }
    for (int off = 32; off > 0; off >>= 1) {
        qn2 += __shfl_xor(qn2, off);
    }
    const float cn2 = __uint_as_float(*p.max_norm_bits);
    const float u = 5.9604644775390625e-8F;
    float eps;
    if constexpr (METRIC == VSAG_AMD_METRIC_L2) {
        const float reach = sqrtf(qn2) + sqrtf(cn2);
        eps = 2.0F * static_cast<float>(p.dim + 8) * u * reach * reach * 1.001F;
    } else {
        eps = 2.0F * static_cast<float>(p.dim + 8) * u * (sqrtf(qn2) * sqrtf(cn2) + 1.0F) * 1.001F;
    }
    odd = odd || !(eps < 1.0e30F) || !(vmax < 1.0e30F) || !(vmin > -1.0e30F);
    const uint32_t qi[1] = {static_cast<uint32_t>(q)};
    if (__ballot(odd) != 0 || p.k > p.n) {
        table_redo<METRIC>(a, p.n, p.ntiles, p.k, qi[0], p.ids + q * p.k, p.dists + q * p.k, kInfKey, pool, lane);
        return;
    }
    // Any value with at least k table values at or below it serves as a_k (a larger one only admits more): 256 bins
    // between the smallest and the largest value, the first bin at which the running count reaches k, and two bins more
    // for the rounding of the binning itself.
    const float width = (vmax - vmin) * (1.0F / 256.0F);
    const float inv_width = width > 0.0F ? 1.0F / width : 0.0F;
    for (uint32_t b = lane; b < 256; b += kWave) {
        hist[b] = 0;
    }
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = static_cast<uint32_t>(i) * kWave + lane;
        if (c < p.n) {
            const float f = (val[i] - vmin) * inv_width;
            atomicAdd(&hist[f < 255.0F ? static_cast<uint32_t>(f) : 255U], 1U);
        }
    }
    wave_lds_fence();
    uint32_t bin;
    {
        const uint32_t h0 = hist[4 * lane], h1 = hist[4 * lane + 1], h2 = hist[4 * lane + 2], h3 = hist[4 * lane + 3];
        uint32_t incl = h0 + h1 + h2 + h3;
        const uint32_t mine = incl;
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(incl, off);
            incl += lane >= static_cast<uint32_t>(off) ? o : 0U;
        }
        const uint64_t reached = __ballot(incl >= p.k);
        const uint32_t owner = static_cast<uint32_t>(__builtin_ctzll(reached));  // k <= n: some lane reaches it
        uint32_t before = __shfl(incl - mine, static_cast<int>(owner));
        const uint32_t o0 = __shfl(h0, static_cast<int>(owner)), o1 = __shfl(h1, static_cast<int>(owner)),
                       o2 = __shfl(h2, static_cast<int>(owner));
        bin = 4 * owner;
        if (before + o0 < p.k) {
            before += o0;
            ++bin;
            if (before + o1 < p.k) {
                before += o1;
                ++bin;
                if (before + o2 < p.k) {
                    ++bin;
                }
            }
        }
    }
    const float kth = vmin + static_cast<float>(bin + 3) * width;  // the upper edge of bin + 2
    // rounded up: what is added here only admits more
    const float thr = (kth + 2.0F * eps) + fabsf(kth + 2.0F * eps) * 4.0F * u;
    uint32_t count = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = static_cast<uint32_t>(i) * kWave + lane;
        const bool pass = c < p.n && val[i] <= thr;
        const uint64_t mask = __ballot(pass);
        const uint32_t at = count + mask_rank(mask);
        if (pass && at < kTablePool) {
            cand[at] = c;
        }
        count += static_cast<uint32_t>(__popcll(mask));
    }
    wave_lds_fence();
    if (count > kTablePool) {
        // many codes at nearly the same distance: the full scan sorts it out
        table_redo<METRIC>(a, p.n, p.ntiles, p.k, qi[0], p.ids + q * p.k, p.dists + q * p.k, kInfKey, pool, lane);
        return;
    }
    const QueryRows<1> qrows = query_rows<1>(a, qi);
    uint32_t sorted = kWave;  // the power of two from the candidates on
    while (sorted < count) {
        sorted <<= 1;
    }
    for (uint32_t base = 0; base < sorted; base += kWave) {
        if (base >= count) {
            pool[base + lane] = kInfKey;
            continue;
        }
        const bool have = base + lane < count;
        const uint32_t slot = have ? cand[base + lane] : 0U;
        const uint4* code = p.rows + static_cast<uint64_t>(slot) * p.row_granules;
        Acc<VSAG_AMD_KIND_FP32, 1> acc;
        acc_reset(acc);
        constexpr uint32_t kAhead = 8;
        for (uint32_t j0 = 0; j0 < a.G; j0 += kAhead) {
            uint4 c4[kAhead];
#pragma unroll
            for (uint32_t v = 0; v < kAhead; ++v) {
                const uint32_t j = j0 + v < a.G ? j0 + v : a.G - 1;
                c4[v] = code[j];
            }
#pragma unroll
            for (uint32_t v = 0; v < kAhead; ++v) {
                if (j0 + v < a.G) {
                    accumulate_granule<VSAG_AMD_KIND_FP32, METRIC, 1>(a, qrows, j0 + v, c4[v], acc);
                }
            }
        }
        float d[1];
        finish_distances<VSAG_AMD_KIND_FP32, METRIC, 1>(a, qi, slot, acc, d);
        pool[base + lane] = have ? make_key(d[0], slot) : kInfKey;
    }
    wave_lds_fence();
    wave_bitonic_sort(pool, sorted, lane);
    for (uint32_t i = lane; i < p.k; i += kWave) {
        const uint64_t key64 = i < sorted ? pool[i] : kInfKey;
        p.ids[q * p.k + i] = key64 == kInfKey ? VSAG_AMD_INVALID_ID : static_cast<uint32_t>(key64);
        p.dists[q * p.k + i] = key64 == kInfKey ? __builtin_inff() : ordered_to_float(static_cast<uint32_t>(key64 >> 32));
    }
}

template <int METRIC>
static void
launch_table_select(uint64_t codes, dim3 grid, hipStream_t st, const ScanArgs& a, const TableSelectArgs& p) {
    if (codes <= 1024) {
        hipLaunchKernelGGL((table_select_kernel<METRIC, 16>), grid, dim3(kWave), 0, st, a, p);
    } else if (codes <= 2048) {
        hipLaunchKernelGGL((table_select_kernel<METRIC, 32>), grid, dim3(kWave), 0, st, a, p);
    } else if (codes <= 4096) {
        hipLaunchKernelGGL((table_select_kernel<METRIC, 64>), grid, dim3(kWave), 0, st, a, p);
    } else {
        hipLaunchKernelGGL((table_select_kernel<METRIC, 128>), grid, dim3(kWave), 0, st, a, p);
    }
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
    CallPlan cp;
    make_call_plan(s, nq, k, &cp);
    Carver c(nullptr, 0);
    ScanBuffers b;
    return carve_scan(c, cp, nq, k, &b) + 256;
}

extern "C" int
vsag_amd_flat_scan_topk(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
                        uint32_t* ids_dev, float* dists_dev, void* workspace_dev, size_t workspace_bytes,
                        void* stream) {
    return vsag_amd_flat_scan_topk_ex(s, queries_dev, nq, k, nullptr, ids_dev, dists_dev, workspace_dev,
                                      workspace_bytes, stream);
}

namespace {

int flat_scan_call(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
                   const vsag_amd_search_options_t* options, uint32_t* ids_dev, float* dists_dev, void* workspace_dev,
                   size_t workspace_bytes, void* stream);

// One streaming launch over tiles [tile0, tile_end), writing partial lists slot0, slot0 + 1, ...
int
run_streaming(const vsag_amd_store* s, const ScanPlan& p, const ScanArgs& a, const ScanBuffers& b, uint64_t nq,
              uint32_t k, const vsag_amd_search_options_t* options, uint64_t tile0, uint64_t tile_end, uint32_t slot0,
              uint32_t nslots, const uint32_t* gate, hipStream_t st) {
    FlatArgs f{};
    f.n = s->n;
    f.tile0 = tile0;
    f.tile_end = tile_end;
    f.tiles_per_chunk = p.tiles_per_chunk;
    f.nq = nq;
    f.k = k;
    f.S = p.S;
    f.nslots = nslots;
    f.slot0 = slot0;
    f.gate = gate;
    f.bound = b.bound;
    f.partial = b.partial;
    f.partial_cnt = b.partial_cnt;
    f.seed = p.seeded ? b.seed : nullptr;
    f.deny = options != nullptr ? options->deny_bits_dev : nullptr;
    return launch_flat(s, p, a, f, st);
}

}  // namespace

extern "C" int
vsag_amd_flat_scan_topk_ex(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
                           const vsag_amd_search_options_t* options, uint32_t* ids_dev, float* dists_dev,
                           void* workspace_dev, size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    return flat_scan_call(s, queries_dev, nq, k, options, ids_dev, dists_dev, workspace_dev, workspace_bytes, stream);
}

namespace {

// The whole flat scan of one call on `stream`, with every intermediate buffer carved out of the given workspace.
int
flat_scan_call(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
               const vsag_amd_search_options_t* options, uint32_t* ids_dev, float* dists_dev, void* workspace_dev,
               size_t workspace_bytes, void* stream) {
    VA_TRY(check_scan_call(s, nq, k));
    VA_CHECK_ARG(s->nlist == 0, "flat scan on a posting-list store");
    VA_CHECK_ARG(queries_dev && ids_dev && dists_dev, "null query / output pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    CallPlan cp;
    make_call_plan(s, nq, k, &cp);
    Carver c(workspace_dev, workspace_bytes);
    ScanBuffers b;
    carve_scan(c, cp, nq, k, &b);
    if (!c.ok() && cp.one) {
        // A workspace sized without the one-query route's distance array (the fixed scratch of the entry point that
        // allocates nothing): the query streams like a batch.
        cp.one = false;
        c = Carver(workspace_dev, workspace_bytes);
        carve_scan(c, cp, nq, k, &b);
    }
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    // A pre-filter or a radius goes the streaming way (the prefilter knows neither).
    const bool plain = options == nullptr || (options->deny_bits_dev == nullptr && options->use_radius == 0);
    const bool contraction = cp.contraction && plain;
    const ScanPlan& p = cp.all;

    VA_TRY(prepare_queries(s, queries_dev, nq, p.nq_pad, p.ql, b.qtab, b.qmeta, b.qcodes, st));
    if (cp.table && plain) {
        const ScanArgs ta = make_scan_args(s, p.ql, b.qtab, b.qmeta);
        const uint64_t slots = cp.table_ld;
        const bool l2 = s->metric == VSAG_AMD_METRIC_L2;
        uint32_t* max_bits = reinterpret_cast<uint32_t*>(b.table_norms + slots);
        const uint32_t row_words = p.ql.qstride;  // a multiple of 16: the rows of the query table, zero behind the dimension
        hipLaunchKernelGGL(table_rows_kernel, dim3(static_cast<uint32_t>(div_up(slots * (row_words / 4), 256))), dim3(256),
                           0, st, s->tiles, s->G, row_words / 4, s->n, slots, b.table_rows, max_bits);
        VA_TRY(launch_row_sqnorms(b.table_rows, slots, row_words, b.table_norms, max_bits, st));
        timing_begin(st);
        VA_TRY(launch_row_products(b.table_rows, slots, reinterpret_cast<const float*>(b.qtab), static_cast<uint32_t>(nq),
                                   row_words, l2 ? b.table_norms : nullptr, l2 ? -2.0F : -1.0F, b.table, cp.table_ld, st));
        TableSelectArgs tp{b.table, cp.table_ld, nq, s->n, s->ntiles, k, row_words, max_bits, ids_dev, dists_dev,
                           reinterpret_cast<const uint4*>(b.table_rows), row_words / 4};
        const dim3 grid(static_cast<uint32_t>(nq));
        if (l2) {
            launch_table_select<VSAG_AMD_METRIC_L2>(slots, grid, st, ta, tp);
        } else {
            launch_table_select<VSAG_AMD_METRIC_IP>(slots, grid, st, ta, tp);
        }
        timing_end(st);
        VA_HIP(hipGetLastError());
        tl_last_tile = 64;
        tl_last_passes = nq;
        return 0;
    }
    if (cp.one && s->ntiles == cp.one_tiles) {
        const ScanArgs oa = make_scan_args(s, p.ql, b.qtab, b.qmeta);
        VA_TRY(launch_one_query(s, oa, k, options, b.one_dist, b.one_mins, ids_dev, dists_dev, st));
        tl_last_tile = 1;
        tl_last_passes = 1;
        tl_last_bytes = s->ntiles * s->G * kWave * kGranule;
        return 0;
    }
    const uint64_t nseed = b.seed != nullptr ? nq * k : 0;
    hipLaunchKernelGGL(reset_queries_kernel, dim3(static_cast<uint32_t>(div_up(nq > nseed ? nq : nseed, 256))), dim3(256),
                       0, st, b.bound, initial_bound(options), nq, b.seed, nseed);
    ScanArgs a = make_scan_args(s, p.ql, b.qtab, b.qmeta);
    uint32_t nslots = 0;
    if (s->ntiles == 0) {
        // An empty store has no lists to read.
    } else if (!contraction) {
        nslots = static_cast<uint32_t>(p.chunks * p.waves);
        timing_begin(st);
        VA_TRY(run_streaming(s, p, a, b, nq, k, options, 0, s->ntiles, 0, nslots, nullptr, st));
        timing_end(st);
        tl_last_tile = p.T;
        tl_last_passes = p.groups;
    } else {
        const uint32_t slots_prefix = static_cast<uint32_t>(cp.prefix.chunks * cp.prefix.waves);
        const uint32_t slots_rest = static_cast<uint32_t>(cp.rest.chunks * cp.rest.waves);
        const uint32_t levels = static_cast<uint32_t>(cp.levels);
        nslots = slots_prefix + levels + slots_rest;
        // The gated launch leaves the lists of most queries untouched: they must read as empty.  No query has
        // overflowed yet.
        hipLaunchKernelGGL(fill_words2_kernel, dim3(static_cast<uint32_t>(div_up(nq * nslots, 256))), dim3(256), 0, st,
                           b.partial_cnt, nq * nslots, b.gate, nq);
        VA_TRY(run_streaming(s, cp.prefix, a, b, nq, k, nullptr, 0, cp.prefix_tiles, 0, nslots, nullptr, st));
        for (uint32_t l = 0; l < levels; ++l) {
            // The lists so far each know the k-th distance of their own part only; the k-th of everything before
            // this level (a merge into the output arrays, which the final merge overwrites) is the bound to
            // filter it with.
            VA_TRY(launch_merge_partials(b.partial, b.partial_cnt, b.bound, slots_prefix + l, nslots, k, p.S, nq, ids_dev,
                                         dists_dev, st));
            // (The int8 route lowers the bounds itself from its second level on, in the launch that renews its
            // thresholds.)
            const bool folded = cp.int8 && !cp.rb && l > 0;
            if (!folded) {
                hipLaunchKernelGGL(tighten_bound_kernel, dim3(static_cast<uint32_t>(div_up(nq, 256))), dim3(256), 0, st,
                                   dists_dev, k, nq, b.bound);
            }
            if (!cp.int8 && !cp.rb) {
                hipLaunchKernelGGL(fill_words2_kernel, dim3(static_cast<uint32_t>(div_up(nq, 256))), dim3(256), 0, st,
                                   b.cand_cnt, nq, static_cast<uint32_t*>(nullptr), 0);
            }
            VA_TRY(launch_prefilter(s, a, nq, k, p.S, cp.level_begin[l], cp.level_begin[l + 1], b.bound, b.tau, b.cand,
                                    b.cand_cnt, cp.cap, b.partial, b.partial_cnt, nslots, slots_prefix, slots_prefix + l,
                                    b.gate, b.q8, b.q8_u, cp.sub_lists[l], cp.sub_cap[l], folded ? dists_dev : nullptr,
                                    st));
        }
        VA_TRY(run_streaming(s, cp.rest, a, b, nq, k, nullptr, cp.prefix_tiles, s->ntiles, slots_prefix + levels, nslots,
                             b.gate, st));
        tl_last_tile = cp.int8 ? 256 : 128;  // queries per pass of the contraction
        tl_last_passes = div_up(nq, cp.int8 ? 256 : 128);
    }
    VA_TRY(launch_merge_partials(b.partial, b.partial_cnt, b.bound, nslots, nslots, k, p.S, nq, ids_dev, dists_dev, st));
    // Code bytes under the timed kernel: the whole store, or the last (by far the largest) level of the contraction.
    const uint64_t timed_tiles = contraction ? s->ntiles - cp.level_begin[cp.levels - 1] : s->ntiles;
    tl_last_bytes = timed_tiles * s->G * kWave * kGranule;
    return 0;
}

}  // namespace

// ---- the flat scan for callers that cannot allocate ------------------------------------------------------------
// The intermediate buffers of a scan (query tables, bounds, seed rows, counted partial lists, candidate lists)
// normally sit in a workspace the caller allocates.  Code under HIP graph capture, tight serving loops and
// harnesses that forbid hipMalloc cannot do that: for them the library keeps one scratch array of fixed size in
// its own device image.  Every GPU the library runs on holds its own copy at its own address until the process
// ends; the address is looked up once per device with that device current.  All calls on one GPU share the array
// and it keeps the last call's contents: every buffer carved from it is (re)initialised by the call that uses
// it, and two calls that overlap on one GPU race.
constexpr size_t kStaticScratchBytes = 32ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxScratchDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxScratchDevices] = {};
static std::mutex g_scratch_mutex;

namespace vsag_amd {
// Looks up the device address of `scratch` on `device`, which must be the current device.
int
static_scratch_setup(int device) {
    VA_CHECK_ARG(device >= 0 && device < kMaxScratchDevices, "device %d out of range [0, %d)", device, kMaxScratchDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device].load(std::memory_order_acquire) != nullptr) {
        return 0;
    }
    void* ptr = nullptr;
    VA_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) {
        return fail(VSAG_AMD_INTERNAL_ERROR, "the library's scratch array has no address on device %d", device);
    }
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return 0;
}
bool timing_suppress(bool off);
}  // namespace vsag_amd

extern "C" size_t
vsag_amd_flat_scan_noalloc_max_bytes(void) {
    return kStaticScratchBytes;
}

extern "C" int
vsag_amd_flat_scan_topk_noalloc(const vsag_amd_store_t* s, const float* queries_dev, uint64_t nq, uint32_t k,
                                const vsag_amd_search_options_t* options, uint32_t* ids_dev, float* dists_dev,
                                void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_scan_call(s, nq, k));
    int device = 0;
    VA_HIP(hipGetDevice(&device));
    VA_CHECK_ARG(device >= 0 && device < kMaxScratchDevices, "device %d out of range [0, %d)", device, kMaxScratchDevices);
    if (g_scratch_ptr[device].load(std::memory_order_acquire) == nullptr) {
        // A device the library was not initialised on: first call there.
        VA_TRY(static_scratch_setup(device));
    }
    void* const scratch_dev = g_scratch_ptr[device].load(std::memory_order_acquire);
    const size_t need = vsag_amd_flat_scan_workspace_bytes(s, nq, k);
    VA_CHECK_ARG(need != 0 && need <= kStaticScratchBytes,
                 "this scan needs %zu bytes of scratch memory, the library's own array holds %zu: send fewer queries "
                 "per call or use vsag_amd_flat_scan_topk_ex with a workspace",
                 need, kStaticScratchBytes);
    // The measurement hook creates events on first use: not in this call.
    const bool was = timing_suppress(true);
    const int rc = flat_scan_call(s, queries_dev, nq, k, options, ids_dev, dists_dev, scratch_dev,
                                  kStaticScratchBytes, stream);
    timing_suppress(was);
    return rc;
}

namespace vsag_amd {
int
scan_contraction_mode(const vsag_amd_store* s) {
    return prefilter_mode(s);
}

// What vsag_amd_last_scan_info reports, for the posting-list scan.
void
note_last_scan(int query_tile, uint64_t passes, uint64_t bytes_per_pass) {
    tl_last_tile = query_tile;
    tl_last_passes = passes;
    tl_last_bytes = bytes_per_pass;
}
}  // namespace vsag_amd

extern "C" int
vsag_amd_set_scan_contraction(int mode) {
    VA_CHECK_ARG(mode >= -1 && mode <= 2,
                 "mode must be -1 (never), 0 (when it pays), 1 (whenever supported) or 2 (1 on the fp32 matrix cores)");
    g_prefilter_mode = mode;
    return 0;
}

extern "C" int
vsag_amd_store_set_scan_contraction(vsag_amd_store_t* s, int mode) {
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(mode >= -2 && mode <= 2, "mode must be -2 (follow the process-wide setting), -1, 0, 1 or 2");
    s->contraction_mode = mode;
    return 0;
}

extern "C" int
vsag_amd_store_set_scan_tuning(vsag_amd_store_t* s, int query_tile, int base_chunks) {
    VA_CHECK_ARG(s != nullptr, "store is null");
    VA_CHECK_ARG(query_tile == -1 || query_tile == 0 || query_tile == 1 || query_tile == 2 || query_tile == 4 ||
                     query_tile == 8,
                 "query_tile must be -1 (follow the process-wide setting), 0, 1, 2, 4 or 8");
    VA_CHECK_ARG(base_chunks >= -1 && base_chunks <= 65535, "base_chunks must be in [-1, 65535]");
    s->tile_override = query_tile;
    s->chunk_override = base_chunks;
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
