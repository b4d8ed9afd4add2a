// One query per call against a large flat store (the calling pattern of the reference and of its evaluator:
// BruteForce::SearchWithRequest, src/algorithm/bruteforce/bruteforce.cpp:481-597, one query x every code).
//
// The batched kernel of scan.hip keeps a selector per (wave, query) and shares a bound between waves; with a single
// query all waves start cold together and most of a 50 us launch is that bookkeeping, not bytes.  Here the pass over
// the codes does no selection at all: every workgroup walks its own run of tiles (a wave a quarter of it), writes the
// (ordered) distance of every code and leaves the smallest (distance, id) key of its run.  The runs are disjoint, so the k-th smallest of those
// minima is reached by k different codes -- a valid bound -- and exactly k runs have a minimum at or below it (keys are
// unique): every code of the result lies in one of those k runs.  A second, one-workgroup launch ranks the minima,
// re-reads the distances of those k runs, keeps what the bound admits and ranks that.  The distances are the ones
// accumulate_granule / finish_distances give the batched kernel, in the same order, so both routes return the same
// bits.
#include "distance.h"
#include "store.h"
#include "topk.h"

namespace vsag_amd {

constexpr uint32_t kOneMaxRuns = 2048;      // minima the selecting workgroup ranks in LDS
constexpr uint32_t kOneMinRunTiles = 16;    // a run = the tiles of one workgroup of the pass: four waves, four tiles each
constexpr uint32_t kOneSurvivors = 2048;    // keys at or below the bound the selecting workgroup ranks in LDS
constexpr uint32_t kOneMaxK = 32;           // every round of the selection shrinks the keys by 64 / k

struct OneArgs {
    uint64_t n, ntiles;
    uint32_t run_tiles;       // tiles per workgroup, a multiple of four
    uint32_t runs;
    const uint32_t* deny;
    uint32_t* dist;           // ordered distance per tile slot (0xFFFFFFFF: no code, or denied)
    uint64_t* mins;           // smallest key per run
};

bool
one_query_supports(const vsag_amd_store* s, uint64_t nq, uint32_t k) {
    return nq == 1 && s->nlist == 0 && k <= kOneMaxK && s->ntiles >= 1024;
}

uint32_t
one_query_run_tiles(const vsag_amd_store* s) {
    const uint64_t t = div_up(div_up(s->ntiles, static_cast<uint64_t>(kOneMaxRuns)), 4) * 4;
    return static_cast<uint32_t>(t < kOneMinRunTiles ? kOneMinRunTiles : t);
}

template <int KIND, int METRIC>
__global__ void __launch_bounds__(256)
one_query_distances_kernel(ScanArgs a, OneArgs o) {
    __shared__ uint64_t wave_min[4];
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6;
    const uint32_t wave_tiles = o.run_tiles / 4;
    uint64_t tile_begin = static_cast<uint64_t>(blockIdx.x) * o.run_tiles + wave * wave_tiles;
    uint64_t tile_end = tile_begin + wave_tiles;
    if (tile_end > o.ntiles) {
        tile_end = o.ntiles;
    }
    if (tile_begin > tile_end) {
        tile_begin = tile_end;
    }
    const uint32_t qidx[1] = {0};
    const QueryRows<1> qrows = query_rows<1>(a, qidx);
    constexpr int GROUP = 8;
    constexpr bool OVERLAP = KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32;
    TileStream<GROUP, OVERLAP> cur{a.tiles, lane, tile_begin, tile_end, 1, 0, a.G};
    TileStream<GROUP, OVERLAP> nxt = cur;
    uint4 buf_a[GROUP], buf_b[GROUP];
    if (cur.valid()) {
        cur.load(buf_a, cur.tile);
    }
    Acc<KIND, 1> acc;
    acc_reset(acc);
    uint64_t best = kInfKey;
    auto consume = [&](const uint4(&regs)[GROUP]) {
        const uint32_t first = cur.first();
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const uint32_t g = first + u;
            if (g >= cur.j0 && g < a.G) {
                accumulate_granule<KIND, METRIC, 1>(a, qrows, g, regs[u], acc);
            }
        }
        if (cur.j0 + GROUP < a.G) {
            return;
        }
        const uint64_t id = cur.tile * kWave + lane;
        float d[1];
        finish_distances<KIND, METRIC, 1>(a, qidx, id, acc, d);
        acc_reset(acc);
        const bool valid = id < o.n && !denied(o.deny, id);
        const uint32_t od = valid ? float_to_ordered(d[0]) : 0xFFFFFFFFU;
        o.dist[id] = od;
        const uint64_t key = od == 0xFFFFFFFFU ? kInfKey : (static_cast<uint64_t>(od) << 32) | static_cast<uint32_t>(id);
        best = key < best ? key : best;
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
    for (int off = 32; off > 0; off >>= 1) {
        const uint64_t other = __shfl_xor(best, off);
        best = other < best ? other : best;
    }
    if (lane == 0) {
        wave_min[wave] = best;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < 4; ++w) {
            best = wave_min[w] < best ? wave_min[w] : best;
        }
        o.mins[blockIdx.x] = best;
    }
}

struct OneSelectArgs {
    const uint64_t* mins;
    const uint32_t* dist;
    uint32_t runs, run_tiles;
    uint64_t ntiles;
    uint32_t k;
    uint32_t radius;  // ordered; 0xFFFFFFFF: none
    uint32_t* ids;
    float* dists;
};

// rank[i] = how many of keys[0, n) are smaller than keys[i], for the keys this thread owns (i = tid, tid + 1024, ...):
// every lane reads the same LDS word at a time (a broadcast), so n reads rank one key per thread with no barrier and no
// sorting network.  Keys with rank < limit go to out[rank] (distinct keys have distinct ranks).
__device__ inline void
rank_into(const uint64_t* keys, uint32_t n, uint64_t* out, uint32_t limit) {
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const uint64_t mine = keys[i];
        uint32_t rank = 0;
        const uint4* pairs = reinterpret_cast<const uint4*>(keys);
#pragma unroll 8
        for (uint32_t j = 0; j < n / 2; ++j) {
            const uint4 v = pairs[j];
            const uint64_t a = (static_cast<uint64_t>(v.y) << 32) | v.x, b = (static_cast<uint64_t>(v.w) << 32) | v.z;
            rank += (a < mine ? 1U : 0U) + (b < mine ? 1U : 0U);
        }
        if ((n & 1U) != 0 && keys[n - 1] < mine) {
            ++rank;
        }
        if (rank < limit) {
            out[rank] = mine;
        }
    }
}

__global__ void __launch_bounds__(1024)
one_query_select_kernel(OneSelectArgs o) {
    __shared__ __align__(16) uint64_t keys[kOneMaxRuns];
    __shared__ __align__(16) uint64_t sv[kOneSurvivors];
    __shared__ uint64_t best_k[kOneMaxK];
    __shared__ uint32_t nsv;
    __shared__ uint64_t wave_best[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63U, wave = tid >> 6;
    const uint32_t k = o.k;
    // The k smallest minima.  Ranking all of them against each other is runs^2 comparisons on one compute unit; so
    // first, round by round, every group of 64 keys (a wave's worth) keeps its own k smallest -- the k smallest of all
    // are among them -- until at most 256 keys are left.
    uint32_t n = (o.runs + 63U) / 64U * 64U;
    for (uint32_t i = tid; i < n; i += blockDim.x) {
        keys[i] = i < o.runs ? o.mins[i] : kInfKey;
    }
    if (tid == 0) {
        nsv = 0;
    }
    uint64_t* src = keys;
    uint64_t* dst = sv;
    while (n > 256) {
        const uint32_t groups = n / 64;
        const uint32_t kept = (groups * k + 63U) / 64U * 64U;
        __syncthreads();
        for (uint32_t i = tid; i < kept; i += blockDim.x) {
            dst[i] = kInfKey;
        }
        __syncthreads();
        for (uint32_t g = wave; g < groups; g += 16) {
            const uint64_t mine = src[g * 64 + lane];
            uint32_t rank = 0;
            const uint4* pairs = reinterpret_cast<const uint4*>(src + g * 64);
#pragma unroll 8
            for (uint32_t j = 0; j < 32; ++j) {
                const uint4 v = pairs[j];
                const uint64_t a = (static_cast<uint64_t>(v.y) << 32) | v.x, b = (static_cast<uint64_t>(v.w) << 32) | v.z;
                rank += (a < mine ? 1U : 0U) + (b < mine ? 1U : 0U);
            }
            if (rank < k && mine != kInfKey) {
                dst[g * k + rank] = mine;
            }
        }
        uint64_t* t = src;
        src = dst;
        dst = t;
        n = kept;
    }
    __syncthreads();
    for (uint32_t i = tid; i < k; i += blockDim.x) {
        best_k[i] = kInfKey;
    }
    __syncthreads();
    rank_into(src, n, best_k, k);
    __syncthreads();
    // The k-th smallest minimum (with fewer than k runs holding a code: nothing is excluded), and the radius.
    uint64_t bound = best_k[k - 1];
    const uint64_t ball = (static_cast<uint64_t>(o.radius) << 32) | 0xFFFFFFFFULL;
    if (o.radius != 0xFFFFFFFFU && ball < bound) {
        bound = ball;
    }
    // The runs whose minimum the bound admits: the first of the sorted minima, k at most.
    const uint32_t ncand = k;
    __syncthreads();
    for (uint32_t i = tid; i < ncand; i += blockDim.x) {
        keys[i] = best_k[i];
    }
    __syncthreads();
    const uint32_t run_codes = o.run_tiles * kWave;
    // What the bound admits out of the runs whose minimum it admits.  Eight runs at a time, a thread one code of each:
    // the eight loads are issued together, before any of them is looked at.
    const uint64_t nslots = o.ntiles * kWave;
    for (uint32_t c0 = 0; c0 < ncand; c0 += 8) {
        for (uint32_t off = tid; off < run_codes; off += blockDim.x) {
            uint32_t od[8];
            uint64_t at[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                const uint64_t key = c0 + u < ncand ? keys[c0 + u] : kInfKey;
                const bool admitted = key != kInfKey && key <= bound;
                at[u] = static_cast<uint64_t>(static_cast<uint32_t>(key) / run_codes) * run_codes + off;
                od[u] = admitted && at[u] < nslots ? o.dist[at[u]] : 0xFFFFFFFFU;
            }
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                const uint64_t kk = (static_cast<uint64_t>(od[u]) << 32) | static_cast<uint32_t>(at[u]);
                if (od[u] != 0xFFFFFFFFU && kk <= bound) {
                    const uint32_t pos = atomicAdd(&nsv, 1U);
                    if (pos < kOneSurvivors) {
                        sv[pos] = kk;
                    }
                }
            }
        }
    }
    __syncthreads();
    const uint32_t total = nsv;
    if (total <= kOneSurvivors) {
        for (uint32_t i = tid; i < k; i += blockDim.x) {
            best_k[i] = kInfKey;
        }
        __syncthreads();
        rank_into(sv, total, best_k, k);
        __syncthreads();
        for (uint32_t i = tid; i < k; i += blockDim.x) {
            const uint64_t key = best_k[i];
            o.ids[i] = key == kInfKey ? VSAG_AMD_INVALID_ID : static_cast<uint32_t>(key);
            o.dists[i] = key == kInfKey ? __builtin_inff() : ordered_to_float(static_cast<uint32_t>(key >> 32));
        }
        return;
    }
    // More admitted keys than the list holds (many equal distances, or nearly everything filtered out): the k best
    // one at a time, each the smallest admitted key above the last one.
    uint64_t last = 0;
    bool have_last = false;
    for (uint32_t r = 0; r < k; ++r) {
        uint64_t best = kInfKey;
        for (uint32_t c = wave; c < ncand; c += 16) {
            const uint64_t key = keys[c];
            if (key == kInfKey || key > bound) {
                break;
            }
            const uint64_t first = static_cast<uint64_t>(static_cast<uint32_t>(key) / run_codes) * run_codes;
            const uint64_t end = first + run_codes < o.ntiles * kWave ? first + run_codes : o.ntiles * kWave;
            for (uint64_t i = first + lane; i < end; i += kWave) {
                const uint32_t od = o.dist[i];
                const uint64_t kk = (static_cast<uint64_t>(od) << 32) | static_cast<uint32_t>(i);
                if (od != 0xFFFFFFFFU && kk <= bound && (!have_last || kk > last) && kk < best) {
                    best = kk;
                }
            }
        }
        for (int off = 32; off > 0; off >>= 1) {
            const uint64_t other = __shfl_xor(best, off);
            best = other < best ? other : best;
        }
        if (lane == 0) {
            wave_best[wave] = best;
        }
        __syncthreads();
        best = wave_best[0];
        for (uint32_t w = 1; w < 16; ++w) {
            best = wave_best[w] < best ? wave_best[w] : best;
        }
        __syncthreads();
        if (tid == 0) {
            o.ids[r] = best == kInfKey ? VSAG_AMD_INVALID_ID : static_cast<uint32_t>(best);
            o.dists[r] = best == kInfKey ? __builtin_inff() : ordered_to_float(static_cast<uint32_t>(best >> 32));
        }
        if (best == kInfKey) {
            for (uint32_t i = r + 1 + tid; i < k; i += blockDim.x) {
                o.ids[i] = VSAG_AMD_INVALID_ID;
                o.dists[i] = __builtin_inff();
            }
            return;
        }
        last = best;
        have_last = true;
    }
}

template <int KIND>
static void
launch_one_m(int metric, dim3 grid, hipStream_t st, const ScanArgs& a, const OneArgs& o) {
    // Cosine stores hold normalised vectors and scan as inner product (RaBitQ has its own formula).
    if (metric == VSAG_AMD_METRIC_L2) {
        hipLaunchKernelGGL((one_query_distances_kernel<KIND, VSAG_AMD_METRIC_L2>), grid, dim3(256), 0, st, a, o);
    } else if (metric == VSAG_AMD_METRIC_COSINE && (KIND == VSAG_AMD_KIND_RABITQ || KIND == kKindRabitqF32)) {
        hipLaunchKernelGGL((one_query_distances_kernel<KIND, VSAG_AMD_METRIC_COSINE>), grid, dim3(256), 0, st, a, o);
    } else {
        hipLaunchKernelGGL((one_query_distances_kernel<KIND, VSAG_AMD_METRIC_IP>), grid, dim3(256), 0, st, a, o);
    }
}

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

// dist: ntiles x 64 words; mins: one_query_runs(s) keys.
int
launch_one_query(const vsag_amd_store* s, const ScanArgs& a, uint32_t k, const vsag_amd_search_options_t* options,
                 uint32_t* dist, uint64_t* mins, uint32_t* ids_dev, float* dists_dev, hipStream_t st) {
    OneArgs o{};
    o.n = s->n;
    o.ntiles = s->ntiles;
    o.run_tiles = one_query_run_tiles(s);
    o.runs = static_cast<uint32_t>(div_up(s->ntiles, static_cast<uint64_t>(o.run_tiles)));
    o.deny = options != nullptr ? options->deny_bits_dev : nullptr;
    o.dist = dist;
    o.mins = mins;
    const dim3 grid(o.runs);
    timing_begin(st);
    switch (s->kind) {
        case VSAG_AMD_KIND_FP32:
            launch_one_m<VSAG_AMD_KIND_FP32>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_SQ8:
            launch_one_m<VSAG_AMD_KIND_SQ8>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_SQ4:
            launch_one_m<VSAG_AMD_KIND_SQ4>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_SQ4_UNIFORM:
            launch_one_m<VSAG_AMD_KIND_SQ4_UNIFORM>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_SQ8_UNIFORM:
            launch_one_m<VSAG_AMD_KIND_SQ8_UNIFORM>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_PQFS:
            launch_one_m<VSAG_AMD_KIND_PQFS>(s->metric, grid, st, a, o);
            break;
        case VSAG_AMD_KIND_RABITQ:
            if (s->query_bits == 32) {
                launch_one_m<kKindRabitqF32>(s->metric, grid, st, a, o);
            } else {
                launch_one_m<VSAG_AMD_KIND_RABITQ>(s->metric, grid, st, a, o);
            }
            break;
        default:
            return fail(VSAG_AMD_INVALID_ARGUMENT, "unknown store kind %d", s->kind);
    }
    timing_end(st);
    VA_HIP(hipGetLastError());
    OneSelectArgs z{};
    z.mins = mins;
    z.dist = dist;
    z.runs = o.runs;
    z.run_tiles = o.run_tiles;
    z.ntiles = s->ntiles;
    z.k = k;
    z.radius = initial_bound(options);
    z.ids = ids_dev;
    z.dists = dists_dev;
    hipLaunchKernelGGL(one_query_select_kernel, dim3(1), dim3(1024), 0, st, z);
    VA_HIP(hipGetLastError());
    return 0;
}

}  // namespace vsag_amd
