// k-means assignment as an fp32 MFMA contraction with a fused argmin, centroid update and Lloyd driver
// (KMeansCluster::find_nearest_one_with_blas / Run, src/impl/cluster/kmeans_cluster.cpp:46-305).
//
// The reference forms distances = -2 C X^T with SGEMM into a k x 65536 buffer, then makes a second pass
// adding ||c||^2 and taking std::min_element per row.  Here one kernel does both: a workgroup owns a
// 128-row tile of X and walks the centroid tiles of its group; v_mfma_f32_32x32x2_f32 accumulates
// <c_m, x_n> with centroids as the M side and data rows as the N side, so that after the K loop every
// lane holds 16 centroid values of ONE data row and the argmin needs no cross-lane traffic until the
// very end.  Candidates are (ordered distance, centroid index) keys, so the smallest index wins ties
// exactly like std::min_element.
//
// Grid: x = centroid group (tile t belongs to group t % groups, groups <= 8), y = row tile.  Workgroups
// are dealt round-robin to the eight XCDs in x-major order, so one XCD always works on the same
// quarter-to-eighth of the centroids and keeps them in its own L2, while the X tile is what streams.
#include <hipcub/hipcub.hpp>

#include <mutex>
#include <random>
#include <vector>

#include "common.h"

namespace vsag_amd {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;  // centroids per tile
constexpr int BN = 128;  // data rows per tile
constexpr int BK = 32;   // contraction depth per stage
constexpr int kPlane = BM;  // float4 slots per (parity, chunk) plane

// LDS operand layout for one stage: [parity h = k & 1][chunk c = (k >> 1) / 4][row] of float4, element e
// of the float4 is k = 2 (4 c + e) + h.  A lane of the MFMA (row = lane % 32, h = lane / 32) then reads
// its operand for four consecutive k-steps with one conflict-free ds_read_b128.
struct Stage {
    float4 a[2 * 4 * kPlane];
    float4 b[2 * 4 * kPlane];
};

__device__ inline float4
load_row_chunk(const float* base, uint64_t row, uint64_t rows, uint32_t k0, uint32_t dim, bool aligned) {
    float4 v = make_float4(0.0F, 0.0F, 0.0F, 0.0F);
    if (row < rows) {
        const float* p = base + row * dim + k0;
        if (aligned && k0 + 4 <= dim) {
            v = *reinterpret_cast<const float4*>(p);
        } else {
            if (k0 < dim) {
                v.x = p[0];
            }
            if (k0 + 1 < dim) {
                v.y = p[1];
            }
            if (k0 + 2 < dim) {
                v.z = p[2];
            }
            if (k0 + 3 < dim) {
                v.w = p[3];
            }
        }
    }
    return v;
}

// Scatter one global float4 (k = 4g .. 4g+3 of `row`) into the parity planes.
__device__ inline void
stage_store(float4* plane, uint32_t row, uint32_t g, float4 v) {
    uint32_t c = g >> 1, e = (g & 1) * 2;
    float* even = reinterpret_cast<float*>(&plane[(0 * 4 + c) * kPlane + row]) + e;
    float* odd = reinterpret_cast<float*>(&plane[(1 * 4 + c) * kPlane + row]) + e;
    *reinterpret_cast<float2*>(even) = make_float2(v.x, v.z);
    *reinterpret_cast<float2*>(odd) = make_float2(v.y, v.w);
}

__global__ void __launch_bounds__(256, 2)
kmeans_assign_kernel(const float* __restrict__ X, uint64_t n, const float* __restrict__ C, uint32_t k, uint32_t dim,
                     const float* __restrict__ ynorm, unsigned long long* __restrict__ best, uint32_t groups) {
    __shared__ Stage stage[2];  // 64 KiB: two workgroups fit the 160 KiB of a gfx950 CU

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;   // which 64 centroids of the tile
    const uint32_t wn = wave >> 1;  // which 64 data rows of the tile
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.y) * BN;
    const bool aligned = (dim & 3) == 0;
    const uint32_t ktiles = (dim + BK - 1) / BK;
    const uint32_t ctiles = (k + BM - 1) / BM;

    // Loader roles: 1024 float4 per operand per stage, four per thread.
    uint32_t ld_row[4], ld_g[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        uint32_t idx = tid + 256 * r;
        ld_row[r] = idx >> 3;
        ld_g[r] = idx & 7;
    }

    unsigned long long my_best[2] = {~0ull, ~0ull};  // per n-block of this wave, for row l32

    for (uint32_t ct = blockIdx.x; ct < ctiles; ct += groups) {
        const uint64_t c0 = static_cast<uint64_t>(ct) * BM;
        floatx16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0.0F;
                }
            }
        }
        __syncthreads();  // the previous tile's readers of the stages are done
        float4 ra[4], rb[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            ra[r] = load_row_chunk(C, c0 + ld_row[r], k, 4 * ld_g[r], dim, aligned);
            rb[r] = load_row_chunk(X, row0 + ld_row[r], n, 4 * ld_g[r], dim, aligned);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            stage_store(stage[0].a, ld_row[r], ld_g[r], ra[r]);
            stage_store(stage[0].b, ld_row[r], ld_g[r], rb[r]);
        }
        __syncthreads();
        for (uint32_t kt = 0; kt < ktiles; ++kt) {
            const uint32_t cur = kt & 1;
            if (kt + 1 < ktiles) {
                uint32_t k0 = (kt + 1) * BK;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    ra[r] = load_row_chunk(C, c0 + ld_row[r], k, k0 + 4 * ld_g[r], dim, aligned);
                    rb[r] = load_row_chunk(X, row0 + ld_row[r], n, k0 + 4 * ld_g[r], dim, aligned);
                }
            }
            const float4* pa = stage[cur].a + half * 4 * kPlane + wm * 64 + l32;
            const float4* pb = stage[cur].b + half * 4 * kPlane + wn * 64 + l32;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float4 a0 = pa[c * kPlane];
                float4 a1 = pa[c * kPlane + 32];
                float4 b0 = pb[c * kPlane];
                float4 b1 = pb[c * kPlane + 32];
                const float av0[4] = {a0.x, a0.y, a0.z, a0.w};
                const float av1[4] = {a1.x, a1.y, a1.z, a1.w};
                const float bv0[4] = {b0.x, b0.y, b0.z, b0.w};
                const float bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv0[e], acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv1[e], acc[0][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv0[e], acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv1[e], acc[1][1], 0, 0, 0);
                }
            }
            if (kt + 1 < ktiles) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    stage_store(stage[cur ^ 1].a, ld_row[r], ld_g[r], ra[r]);
                    stage_store(stage[cur ^ 1].b, ld_row[r], ld_g[r], rb[r]);
                }
            }
            __syncthreads();
        }
        // Fused argmin: acc[i][j][e] = <c_m, x_n> with m = c0 + wm*64 + i*32 + 8*(e/4) + 4*half + e%4 and
        // n = row0 + wn*64 + j*32 + l32.  m grows with (i, e), so a strict `<` keeps the first minimum.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            float bd = __builtin_inff();
            uint32_t bi = 0xFFFFFFFFU;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    uint32_t ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    bool ok = c0 + ml < k;
                    float dist = (ok ? ynorm[c0 + ml] : 0.0F) + (-2.0F * acc[i][j][e]);
                    if (ok && dist < bd) {
                        bd = dist;
                        bi = static_cast<uint32_t>(c0) + ml;
                    }
                }
            }
            if (bi != 0xFFFFFFFFU) {
                unsigned long long key = make_key(bd, bi);
                if (key < my_best[j]) {
                    my_best[j] = key;
                }
            }
        }
    }
    // Combine the two halves of the wave (they hold different centroids of the same data row), then
    // publish with one 64-bit atomic per row and wave.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        unsigned long long other = __shfl_xor(my_best[j], 32);
        unsigned long long key = other < my_best[j] ? other : my_best[j];
        uint64_t row = row0 + wn * 64 + j * 32 + l32;
        if (half == 0 && row < n && key != ~0ull) {
            atomicMin(&best[row], key);
        }
    }
}

// v or zeros, component by component (a conditional on the whole float4 would go through memory).
__device__ inline float4
keep_if(bool in, float4 v) {
    v.x = in ? v.x : 0.0F;
    v.y = in ? v.y : 0.0F;
    v.z = in ? v.z : 0.0F;
    v.w = in ? v.w : 0.0F;
    return v;
}

// The same contraction for dim % 4 == 0 (every row is a whole number of float4), one (row tile, centroid tile) per
// workgroup of eight waves: 256 data rows x (64 MI) centroids, MI = 2 or 4.  What bounds this kernel next to the matrix
// pipe is the stream of operand tiles from L2 into the CUs, so the tile is as large as LDS and registers allow: one
// workgroup per CU, 16 MI accumulator registers per 32 data rows.
//
// Stages of 16 k travel through a ring of three LDS slots.  In iteration s a wave stores the rows it loaded for
// stage s + 2 (the loads went out an iteration ago), sends the loads for stage s + 3, and contracts stage s; the
// operands of the first MFMAs of stage s + 1 are read from LDS while the last ones of stage s run, so the matrix pipe
// never waits for LDS across the one barrier per stage.  Slot (s + 2) % 3 last held stage s - 1, which every wave
// finished before the barrier that ended iteration s - 1.
//
// LDS layout per slot and operand: four planes of float4, plane g = 2c + h holds for every row the float4 of
// k = 8c + 4h .. 8c + 4h + 3 of the stage.  The contraction runs over all k, so the k a lane feeds to an MFMA step may
// be any bijection as long as both operands use the same one: lane (row, h) takes k = 8c + 4h + e in step 4c + e,
// which makes a global float4 one ds_write_b128 and a lane's operands for four steps one ds_read_b128.  Row r of
// plane g sits in slot r ^ (10 (g & 1) + 4 (g >> 1)): the float4 written by 8 (16) neighbouring lanes, 2 (4) rows of
// all planes, fall into different 16-byte columns of a 128 (256) byte bank period, and a read of 32 consecutive rows
// stays a permutation of 32 consecutive slots.
//
// Grid: one dimension.  Workgroups are dealt round-robin to the eight XCDs, so id % 8 is the XCD; the ids of one XCD
// walk macro tiles of (32 / mc) row tiles x mc centroid tiles, the 32 workgroups that run at the same time on that
// XCD and advance through k together: a k-slice of a row tile or centroid tile is fetched into the XCD's L2 once and
// hit by the other workgroups of its macro row / column.
struct TilePlan {
    uint32_t rtiles, ctiles;
    uint32_t mc_log2;  // macro tile: (32 >> mc_log2) row tiles x (1 << mc_log2) centroid tiles
    uint32_t mcols;    // macro tiles per macro row
    uint64_t ld;       // STORE: floats per row of the output
    float alpha;       // STORE: factor of the product
    uint32_t macros;
};

constexpr int kTileRows = 256;  // data rows per workgroup tile
constexpr int kTileThreads = 512;
constexpr int kStageK = 16;     // contraction depth per stage
constexpr int kRing = 3;

constexpr size_t
tile_lds_bytes(int mi) {
    return kRing * static_cast<size_t>(4 * (64 * mi + kTileRows)) * sizeof(float4);
}

// STORE: instead of the argmin, every product goes out as out[m * plan.ld + n] = (ynorm ? ynorm[n] : 0) + plan.alpha *
// <c_m, x_n> (m a row of C, n a row of X; `best` is that float matrix, ynorm is indexed by rows of X): the table of
// approximate distances a routing call selects from (scan.hip, route_select_kernel).
template <int MI, bool STORE = false>
__global__ void __launch_bounds__(kTileThreads, 1)
kmeans_assign_tile_kernel(const float* __restrict__ X, uint64_t n, const float* __restrict__ C, uint32_t k, uint32_t dim,
                          const float* __restrict__ ynorm, unsigned long long* __restrict__ best, TilePlan plan) {
    constexpr uint32_t TM = 64 * MI;                   // centroids per tile
    constexpr uint32_t kSlot = 4 * (TM + kTileRows);   // float4 per ring slot: A planes, then B planes
    constexpr int RA = MI / 2;                         // float4 of A a thread loads per stage
    extern __shared__ float4 lds[];

    const uint32_t xcd = blockIdx.x & 7;
    const uint32_t local = blockIdx.x >> 3;
    const uint32_t macro = (local >> 5) * 8 + xcd;
    if (macro >= plan.macros) {
        return;
    }
    const uint32_t within = local & 31;
    const uint32_t rt = (macro / plan.mcols) * (32U >> plan.mc_log2) + (within >> plan.mc_log2);
    const uint32_t ct = ((macro % plan.mcols) << plan.mc_log2) + (within & ((1U << plan.mc_log2) - 1));
    if (rt >= plan.rtiles || ct >= plan.ctiles) {
        return;
    }

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave & 1;   // which half of the tile's centroids
    const uint32_t wn = wave >> 1;  // which 64 data rows of the tile
    const uint32_t half = lane >> 5;
    const uint32_t l32 = lane & 31;
    const uint64_t row0 = static_cast<uint64_t>(rt) * kTileRows;
    const uint64_t c0 = static_cast<uint64_t>(ct) * TM;
    const uint32_t stages = (dim + kStageK - 1) / kStageK;

    // Loader: thread (r, g) of 128 x 4 moves float4 g of rows r, r + 128 of both operands (A: one row when the tile
    // has 128 centroids).  Rows past the end repeat the last one: their results are dropped at the end.
    const uint32_t lr = tid >> 2, lg = tid & 3;
    const float* pa[RA];
    const float* pb[2];
#pragma unroll
    for (int r = 0; r < RA; ++r) {
        const uint64_t ca = c0 + lr + 128 * r;
        pa[r] = C + (ca < k ? ca : k - 1) * dim;
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint64_t xb = row0 + lr + 128 * r;
        pb[r] = X + (xb < n ? xb : n - 1) * dim;
    }
    const uint32_t wslot = lr ^ (10 * (lg & 1) + 4 * (lg >> 1));  // + 128 r
    const uint32_t wa = lg * TM + wslot;
    const uint32_t wb = 4 * TM + lg * kTileRows + wslot;
    // Reader: lane (l32, half) takes plane 2c + half, rows wm * 32 MI + 32 i + l32 of A and wn * 64 + 32 j + l32 of B.
    uint32_t ra_off[2], rb_off[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const uint32_t sw = 10 * half + 4 * c;
        ra_off[c] = (2 * c + half) * TM + wm * 32 * MI + (l32 ^ sw);
        rb_off[c] = 4 * TM + (2 * c + half) * kTileRows + wn * 64 + (l32 ^ sw);
    }

    floatx16 acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0.0F;
            }
        }
    }
    float4 ga[RA], gb[2];
    // Loads of stage t; past the last stage they repeat it and what they bring is never read.
    auto load_column = [&](uint32_t t) {
        const uint32_t k0 = (t < stages ? t : stages - 1) * kStageK + 4 * lg;
        return k0 < dim ? k0 : 0;
    };
    auto issue_loads = [&](uint32_t t) {
        const uint32_t col = load_column(t);
#pragma unroll
        for (int r = 0; r < RA; ++r) {
            ga[r] = *reinterpret_cast<const float4*>(pa[r] + col);
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            gb[r] = *reinterpret_cast<const float4*>(pb[r] + col);
        }
    };
    auto store_stage = [&](uint32_t t, float4* slot) {
        const bool in = t * kStageK + 4 * lg < dim;
#pragma unroll
        for (int r = 0; r < RA; ++r) {
            slot[wa + 128 * r] = keep_if(in, ga[r]);
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            slot[wb + 128 * r] = keep_if(in, gb[r]);
        }
    };
    float4 fa[2][MI], fb[2][2];
    // Operand m of 6 (MI = 4) or 4 (MI = 2) of chunk c of a slot into buffer u.
    auto read_operand = [&](const float4* slot, int c, int u, int m) {
        if (m < MI) {
            fa[u][m] = slot[ra_off[c] + 32 * m];
        } else {
            fb[u][m - MI] = slot[rb_off[c] + 32 * (m - MI)];
        }
    };
    // The 2 MI MFMAs of step e of the chunk in buffer u; side(m) runs behind the m-th of them, so that the loads,
    // stores and LDS reads of the pipeline are issued while the matrix pipe works on an MFMA of this wave.
    auto mfma_step = [&](int u, int e, auto side) {
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const float av = e == 0 ? fa[u][i].x : e == 1 ? fa[u][i].y : e == 2 ? fa[u][i].z : fa[u][i].w;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float bv = e == 0 ? fb[u][j].x : e == 1 ? fb[u][j].y : e == 2 ? fb[u][j].z : fb[u][j].w;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                side(2 * i + j);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    auto nothing = [](int) {};
    float4* s0 = lds;              // slot of the stage being contracted
    float4* s1 = lds + kSlot;      // of the next one
    float4* s2 = lds + 2 * kSlot;  // of the one after
    issue_loads(0);
    store_stage(0, s0);
    issue_loads(1);
    store_stage(1, s1);
    issue_loads(2);
    __syncthreads();
#pragma unroll
    for (int m = 0; m < MI + 2; ++m) {
        read_operand(s0, 0, 0, m);
    }
    for (uint32_t st = 0; st < stages; ++st) {
        const bool in = (st + 2) * kStageK + 4 * lg < dim;
        const uint32_t col = load_column(st + 3);
        // chunk 0; the operands of chunk 1 are read behind its first MFMAs
        mfma_step(0, 0, [&](int m) {
            if (m < MI + 2) {
                read_operand(s0, 1, 1, m);
            }
        });
        mfma_step(0, 1, nothing);
        mfma_step(0, 2, nothing);
        mfma_step(0, 3, nothing);
        // chunk 1; behind it the first operands of stage st + 1 (stored an iteration ago, behind the last barrier),
        // then the rows loaded for stage st + 2 go to LDS and the loads of stage st + 3 go out
        mfma_step(1, 0, [&](int m) {
            if (m < MI + 2) {
                read_operand(s1, 0, 0, m);
            }
        });
        mfma_step(1, 1, [&](int m) {
            if (m < RA) {
                s2[wa + 128 * m] = keep_if(in, ga[m]);
            } else if (m < RA + 2) {
                s2[wb + 128 * (m - RA)] = keep_if(in, gb[m - RA]);
            }
        });
        mfma_step(1, 2, [&](int m) {
            if (m < RA) {
                ga[m] = *reinterpret_cast<const float4*>(pa[m] + col);
            } else if (m < RA + 2) {
                gb[m - RA] = *reinterpret_cast<const float4*>(pb[m - RA] + col);
            }
        });
        mfma_step(1, 3, nothing);
        __syncthreads();
        float4* t = s0;
        s0 = s1;
        s1 = s2;
        s2 = t;
    }
    if constexpr (STORE) {
        float* out = reinterpret_cast<float*>(best);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint64_t row = row0 + wn * 64 + j * 32 + l32;
            const float base = row < n && ynorm != nullptr ? ynorm[row] : 0.0F;
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t ml = wm * 32 * MI + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                    if (row < n && c0 + ml < k) {
                        out[(c0 + ml) * plan.ld + row] = base + plan.alpha * acc[i][j][e];
                    }
                }
            }
        }
        return;
    }
    // Fused argmin: acc[i][j][e] = <c_m, x_n> with m = c0 + wm*32*MI + i*32 + 8*(e/4) + 4*half + e%4 and
    // n = row0 + wn*64 + j*32 + l32.  m grows with (i, e), so a strict `<` keeps the first minimum.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        float bd = __builtin_inff();
        uint32_t bi = 0xFFFFFFFFU;
#pragma unroll
        for (int i = 0; i < MI; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t ml = wm * 32 * MI + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                const bool ok = c0 + ml < k;
                const float dist = (ok ? ynorm[c0 + ml] : 0.0F) + (-2.0F * acc[i][j][e]);
                if (ok && dist < bd) {
                    bd = dist;
                    bi = static_cast<uint32_t>(c0) + ml;
                }
            }
        }
        // the two halves of the wave hold different centroids of the same data row
        unsigned long long key = bi != 0xFFFFFFFFU ? make_key(bd, bi) : ~0ull;
        const unsigned long long other = __shfl_xor(key, 32);
        key = other < key ? other : key;
        const uint64_t row = row0 + wn * 64 + j * 32 + l32;
        if (half == 0 && row < n && key != ~0ull) {
            atomicMin(&best[row], key);
        }
    }
}

__global__ void
fill_u64_kernel(unsigned long long* p, unsigned long long v, uint64_t n) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// ||row||^2 for every row; one wave per row.
__global__ void __launch_bounds__(256)
row_sqnorm_kernel(const float* x, uint64_t n, uint32_t dim, float* out) {
    uint64_t row = static_cast<uint64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    uint32_t lane = threadIdx.x & 63;
    if (row >= n) {
        return;
    }
    const float* r = x + row * dim;
    float s = 0.0F;
    for (uint32_t d = lane; d < dim; d += 64) {
        s = fmaf(r[d], r[d], s);
    }
    for (int off = 32; off > 0; off >>= 1) {
        s += __shfl_down(s, off);
    }
    if (lane == 0) {
        out[row] = s;
    }
}

// labels / min distances out of the keys, and the loss: sum over rows of double(float(min + ||x||^2))
// (kmeans_cluster.cpp:279-304).  Block partial sums go to `partial` and are added in block order by the
// last kernel, so the result does not depend on scheduling.
__global__ void __launch_bounds__(256)
kmeans_finalize_kernel(const unsigned long long* best, const float* xnorm, uint64_t n, int32_t* labels,
                       float* min_dist, double* partial) {
    __shared__ double red[4];
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    double v = 0.0;
    if (i < n) {
        unsigned long long key = best[i];
        float md = ordered_to_float(static_cast<uint32_t>(key >> 32));
        labels[i] = static_cast<int32_t>(static_cast<uint32_t>(key));
        if (min_dist != nullptr) {
            min_dist[i] = md;
        }
        v = static_cast<double>(md + xnorm[i]);
    }
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_down(v, off);
    }
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = v;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        partial[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
    }
}

__global__ void
loss_reduce_kernel(const double* partial, uint64_t count, uint64_t n, double* loss) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        double s = 0.0;
        for (uint64_t i = 0; i < count; ++i) {
            s += partial[i];
        }
        *loss = s / static_cast<float>(n);
    }
}

// ------------------------------------------------------------------ centroid update
__global__ void
iota_u32_kernel(uint32_t* p, uint64_t n) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = static_cast<uint32_t>(i);
    }
}

__global__ void
count_labels_kernel(const int32_t* labels, uint64_t n, uint32_t k, uint32_t* counts) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        int32_t l = labels[i];
        if (l >= 0 && static_cast<uint32_t>(l) < k) {
            atomicAdd(&counts[l], 1U);
        }
    }
}

// Exclusive prefix sum of k counts by one workgroup (k is a few thousand).
__global__ void __launch_bounds__(1024)
exclusive_scan_kernel(const uint32_t* counts, uint32_t k, uint32_t* offsets) {
    __shared__ uint32_t sums[1024];
    uint32_t per = (k + blockDim.x - 1) / blockDim.x;
    uint32_t begin = threadIdx.x * per;
    uint32_t end = begin + per < k ? begin + per : k;
    uint32_t s = 0;
    for (uint32_t i = begin; i < end; ++i) {
        s += counts[i];
    }
    sums[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (uint32_t i = 0; i < blockDim.x; ++i) {
            uint32_t t = sums[i];
            sums[i] = run;
            run += t;
        }
        offsets[k] = run;
    }
    __syncthreads();
    uint32_t run = sums[threadIdx.x];
    for (uint32_t i = begin; i < end; ++i) {
        offsets[i] = run;
        run += counts[i];
    }
}

// One workgroup per centroid: mean of its member rows (rows sorted by label, in row order), fp32 running
// sums per dimension.  Empty clusters keep their centroid.
__global__ void __launch_bounds__(256)
centroid_mean_kernel(const float* x, uint32_t dim, const uint32_t* sorted_rows, const uint32_t* offsets,
                     float* centroids, int32_t* counts_out) {
    uint32_t j = blockIdx.x;
    uint32_t begin = offsets[j], end = offsets[j + 1];
    if (threadIdx.x == 0) {
        counts_out[j] = static_cast<int32_t>(end - begin);
    }
    if (end == begin) {
        return;
    }
    float inv = 1.0F / static_cast<float>(end - begin);
    for (uint32_t d0 = 0; d0 < dim; d0 += blockDim.x * 4) {
        uint32_t d = d0 + threadIdx.x * 4;
        float s[4] = {0.0F, 0.0F, 0.0F, 0.0F};
        if (d + 4 <= dim && (dim & 3) == 0) {
            // Eight member rows in flight per thread; the additions keep the row order.
            constexpr uint32_t kAhead = 8;
            for (uint32_t p = begin; p < end; p += kAhead) {
                float4 v[kAhead];
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    uint32_t pp = p + u < end ? p + u : end - 1;
                    v[u] = *reinterpret_cast<const float4*>(x + static_cast<uint64_t>(sorted_rows[pp]) * dim + d);
                }
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    if (p + u < end) {
                        s[0] += v[u].x;
                        s[1] += v[u].y;
                        s[2] += v[u].z;
                        s[3] += v[u].w;
                    }
                }
            }
        } else {
            for (uint32_t p = begin; p < end; ++p) {
                const float* r = x + static_cast<uint64_t>(sorted_rows[p]) * dim;
                for (int e = 0; e < 4; ++e) {
                    if (d + e < dim) {
                        s[e] += r[d + e];
                    }
                }
            }
        }
        for (int e = 0; e < 4; ++e) {
            if (d + e < dim) {
                centroids[static_cast<uint64_t>(j) * dim + d + e] = s[e] * inv;
            }
        }
    }
}

void timing_begin(hipStream_t st);
void timing_end(hipStream_t st);

// out[m * ld + n] = (base ? base[n] : 0) + alpha <c_m, x_n> for the rows x_n of x (nx x dim) and c_m of c (nc x dim), on
// the fp32 matrix cores; dim a multiple of 4, rows 16-byte aligned.
int
launch_row_products(const float* x, uint64_t nx, const float* c, uint32_t nc, uint32_t dim, const float* base, float alpha,
                    float* out, uint64_t ld, hipStream_t st) {
    if ((dim & 3) != 0 || nx == 0 || nc == 0 || nx > (1ull << 20) * kTileRows) {
        return fail(VSAG_AMD_INVALID_ARGUMENT, "row products: the dimension must be a multiple of 4");
    }
    static std::once_flag lds_once;
    static hipError_t lds_rc = hipSuccess;
    std::call_once(lds_once, []() {
        lds_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kmeans_assign_tile_kernel<4, true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(tile_lds_bytes(4)));
    });
    VA_HIP(lds_rc);
    TilePlan plan;
    plan.rtiles = static_cast<uint32_t>(div_up(nx, kTileRows));
    plan.ctiles = (nc + 255) / 256;
    plan.mc_log2 = plan.ctiles >= 8 ? 3 : plan.ctiles >= 4 ? 2 : plan.ctiles >= 2 ? 1 : 0;
    plan.mcols = (plan.ctiles + (1U << plan.mc_log2) - 1) >> plan.mc_log2;
    const uint32_t mrows = (plan.rtiles + (32U >> plan.mc_log2) - 1) / (32U >> plan.mc_log2);
    plan.macros = mrows * plan.mcols;
    plan.ld = ld;
    plan.alpha = alpha;
    const uint32_t per_xcd = (plan.macros + 7) / 8;
    const dim3 grid(per_xcd * 32 * 8);
    hipLaunchKernelGGL((kmeans_assign_tile_kernel<4, true>), grid, dim3(kTileThreads), tile_lds_bytes(4), st, x, nx, c, nc,
                       dim, base, reinterpret_cast<unsigned long long*>(out), plan);
    VA_HIP(hipGetLastError());
    return 0;
}

// The largest finite value of out[0, n) as float bits (norms: not negative, so the bits order like the values); one
// workgroup.
__global__ void __launch_bounds__(1024)
max_norm_kernel(const float* out, uint64_t n, uint32_t* max_bits) {
    __shared__ float part[16];
    float m = 0.0F;
    for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = out[i];
        m = v < __builtin_inff() ? fmaxf(m, v) : m;
    }
    for (int off = 32; off > 0; off >>= 1) {
        m = fmaxf(m, __shfl_xor(m, off));
    }
    if ((threadIdx.x & 63) == 0) {
        part[threadIdx.x >> 6] = m;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < blockDim.x / 64; ++w) {
            m = fmaxf(m, part[w]);
        }
        *max_bits = __float_as_uint(m);
    }
}

// ||row||^2 of nx rows and the largest of them (as float bits).
int
launch_row_sqnorms(const float* x, uint64_t nx, uint32_t dim, float* out, uint32_t* max_bits, hipStream_t st) {
    hipLaunchKernelGGL(row_sqnorm_kernel, dim3(static_cast<uint32_t>(div_up(nx, 4))), dim3(256), 0, st, x, nx, dim, out);
    hipLaunchKernelGGL(max_norm_kernel, dim3(1), dim3(1024), 0, st, out, nx, max_bits);
    VA_HIP(hipGetLastError());
    return 0;
}

struct AssignBuffers {
    float* ynorm;
    float* xnorm;
    unsigned long long* best;
    double* partial;
    double* loss_tmp;
};

static size_t
carve_assign(Carver& c, uint64_t n, uint32_t k, AssignBuffers* b) {
    b->ynorm = c.take<float>(k);
    b->xnorm = c.take<float>(n);
    b->best = c.take<unsigned long long>(n);
    b->partial = c.take<double>(div_up(n, 256));
    b->loss_tmp = c.take<double>(1);
    return c.used;
}

static int
assign_launch(const float* x, uint64_t n, uint32_t dim, const float* cent, uint32_t k, int32_t* labels,
              float* min_dist, double* loss_dev, const AssignBuffers& b, bool have_xnorm, hipStream_t st) {
    hipLaunchKernelGGL(row_sqnorm_kernel, dim3(static_cast<uint32_t>(div_up(k, 4))), dim3(256), 0, st, cent,
                       static_cast<uint64_t>(k), dim, b.ynorm);
    if (!have_xnorm) {
        hipLaunchKernelGGL(row_sqnorm_kernel, dim3(static_cast<uint32_t>(div_up(n, 4))), dim3(256), 0, st, x, n, dim,
                           b.xnorm);
    }
    hipLaunchKernelGGL(fill_u64_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, b.best, ~0ull,
                       n);
    uint32_t ctiles = (k + BM - 1) / BM;
    timing_begin(st);
    if ((dim & 3) == 0) {
        // 256 centroids per tile when there are enough of them to fill it, else 128
        const int mi = k > 384 ? 4 : 2;
        const uint32_t tile_m = 64 * mi;
        static std::once_flag lds_once;
        static hipError_t lds_rc = hipSuccess;
        std::call_once(lds_once, []() {
            lds_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kmeans_assign_tile_kernel<2>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(tile_lds_bytes(2)));
            if (lds_rc == hipSuccess) {
                lds_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kmeans_assign_tile_kernel<4>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(tile_lds_bytes(4)));
            }
        });
        VA_HIP(lds_rc);
        // rows go slab by slab so that the tile count stays far inside the grid limit
        const uint64_t slab_rows = (1ull << 20) * kTileRows;
        for (uint64_t r0 = 0; r0 < n; r0 += slab_rows) {
            const uint64_t rows = n - r0 < slab_rows ? n - r0 : slab_rows;
            TilePlan plan;
            plan.rtiles = static_cast<uint32_t>(div_up(rows, kTileRows));
            plan.ctiles = (k + tile_m - 1) / tile_m;
            plan.mc_log2 = plan.ctiles >= 8 ? 3 : plan.ctiles >= 4 ? 2 : plan.ctiles >= 2 ? 1 : 0;
            plan.mcols = (plan.ctiles + (1U << plan.mc_log2) - 1) >> plan.mc_log2;
            const uint32_t mrows = (plan.rtiles + (32U >> plan.mc_log2) - 1) / (32U >> plan.mc_log2);
            plan.macros = mrows * plan.mcols;
            plan.ld = 0;
            plan.alpha = 0.0F;
            const uint32_t per_xcd = (plan.macros + 7) / 8;
            const dim3 grid(per_xcd * 32 * 8);
            if (mi == 4) {
                hipLaunchKernelGGL(kmeans_assign_tile_kernel<4>, grid, dim3(kTileThreads), tile_lds_bytes(4), st,
                                   x + r0 * dim, rows, cent, k, dim, b.ynorm, b.best + r0, plan);
            } else {
                hipLaunchKernelGGL(kmeans_assign_tile_kernel<2>, grid, dim3(kTileThreads), tile_lds_bytes(2), st,
                                   x + r0 * dim, rows, cent, k, dim, b.ynorm, b.best + r0, plan);
            }
        }
    } else {
        uint32_t groups = ctiles < 8 ? ctiles : 8;
        // grid.y is limited to 65535 row tiles: larger inputs go slab by slab.
        const uint64_t slab_rows = 65535ull * BN;
        for (uint64_t r0 = 0; r0 < n; r0 += slab_rows) {
            uint64_t rows = n - r0 < slab_rows ? n - r0 : slab_rows;
            dim3 grid(groups, static_cast<uint32_t>(div_up(rows, BN)));
            hipLaunchKernelGGL(kmeans_assign_kernel, grid, dim3(256), 0, st, x + r0 * dim, rows, cent, k, dim, b.ynorm,
                               b.best + r0, groups);
        }
    }
    timing_end(st);
    hipLaunchKernelGGL(kmeans_finalize_kernel, dim3(static_cast<uint32_t>(div_up(n, 256))), dim3(256), 0, st, b.best,
                       b.xnorm, n, labels, min_dist, b.partial);
    hipLaunchKernelGGL(loss_reduce_kernel, dim3(1), dim3(64), 0, st, b.partial, div_up(n, 256), n,
                       loss_dev ? loss_dev : b.loss_tmp);
    VA_HIP(hipGetLastError());
    return 0;
}

struct UpdateBuffers {
    uint32_t* counts;
    uint32_t* offsets;
    uint32_t* rows_in;
    uint32_t* rows_out;
    int32_t* keys_out;
    void* sort_tmp;
    size_t sort_tmp_bytes;
};

static size_t
sort_temp_bytes(uint64_t n) {
    size_t bytes = 0;
    // A size query only; a failure leaves 0 and the sort that follows reports it.
    if (hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, static_cast<const int32_t*>(nullptr),
                                           static_cast<int32_t*>(nullptr), static_cast<const uint32_t*>(nullptr),
                                           static_cast<uint32_t*>(nullptr), static_cast<int>(n), 0, 32,
                                           nullptr) != hipSuccess) {
        bytes = 0;
    }
    return bytes;
}

static size_t
carve_update(Carver& c, uint64_t n, uint32_t k, UpdateBuffers* b) {
    b->counts = c.take<uint32_t>(k + 1);
    b->offsets = c.take<uint32_t>(k + 1);
    b->rows_in = c.take<uint32_t>(n);
    b->rows_out = c.take<uint32_t>(n);
    b->keys_out = c.take<int32_t>(n);
    b->sort_tmp_bytes = sort_temp_bytes(n);
    b->sort_tmp = c.take<uint8_t>(b->sort_tmp_bytes);
    return c.used;
}

// Few, short centroids (the 16 centroids of a product-quantizer subspace): sorting the rows by label and giving a
// workgroup to each centroid leaves the machine idle.  Instead a workgroup sums a block of 1024 rows per (centroid,
// dimension) in row order, and a second launch adds the block sums in block order -- the order of the reference's own
// update, which sums per task of 1024 rows and merges the tasks (kmeans_cluster.cpp:108-154).
constexpr uint32_t kSmallUpdateRows = 1024;

__global__ void __launch_bounds__(256)
small_update_partial_kernel(const float* x, const int32_t* labels, uint64_t n, uint32_t dim, uint32_t k, float* psum,
                            uint32_t* pcount) {
    __shared__ int32_t lab[kSmallUpdateRows];
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * kSmallUpdateRows;
    const uint32_t rows = static_cast<uint32_t>(n - row0 < kSmallUpdateRows ? n - row0 : kSmallUpdateRows);
    for (uint32_t r = threadIdx.x; r < rows; r += blockDim.x) {
        lab[r] = labels[row0 + r];
    }
    __syncthreads();
    const uint32_t entries = k * dim;
    for (uint32_t e = threadIdx.x; e < entries; e += blockDim.x) {
        const int32_t c = static_cast<int32_t>(e / dim);
        const uint32_t d = e % dim;
        const float* col = x + row0 * dim + d;
        float s = 0.0F;
        uint32_t cnt = 0;
        for (uint32_t r = 0; r < rows; ++r) {
            if (lab[r] == c) {
                s += col[static_cast<uint64_t>(r) * dim];
                ++cnt;
            }
        }
        psum[static_cast<uint64_t>(blockIdx.x) * entries + e] = s;
        if (d == 0) {
            pcount[static_cast<uint64_t>(blockIdx.x) * k + c] = cnt;
        }
    }
}

__global__ void __launch_bounds__(256)
small_update_final_kernel(const float* psum, const uint32_t* pcount, uint32_t blocks, uint32_t dim, uint32_t k,
                          float* centroids, int32_t* counts_out) {
    const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t entries = k * dim;
    if (e >= entries) {
        return;
    }
    const uint32_t c = e / dim;
    float s = 0.0F;
    uint32_t cnt = 0;
    for (uint32_t b = 0; b < blocks; ++b) {
        const uint32_t bc = pcount[static_cast<uint64_t>(b) * k + c];
        if (bc != 0) {
            s += psum[static_cast<uint64_t>(b) * entries + e];
            cnt += bc;
        }
    }
    if (e % dim == 0) {
        counts_out[c] = static_cast<int32_t>(cnt);
    }
    if (cnt != 0) {
        centroids[e] = s * (1.0F / static_cast<float>(cnt));  // empty clusters keep their centroid
    }
}

static int
update_launch(const float* x, const int32_t* labels, uint64_t n, uint32_t dim, uint32_t k, float* cent,
              int32_t* counts_dev, const UpdateBuffers& b, hipStream_t st) {
    const uint64_t small_blocks = div_up(n, static_cast<uint64_t>(kSmallUpdateRows));
    if (k <= 64 && static_cast<uint64_t>(k) * dim <= 512 && small_blocks * k * dim <= n && small_blocks * k <= n) {
        // the block sums and counts live where the sort of the general path keeps its row lists
        float* psum = reinterpret_cast<float*>(b.rows_in);
        uint32_t* pcount = b.rows_out;
        hipLaunchKernelGGL(small_update_partial_kernel, dim3(static_cast<uint32_t>(small_blocks)), dim3(256), 0, st, x,
                           labels, n, dim, k, psum, pcount);
        hipLaunchKernelGGL(small_update_final_kernel, dim3((k * dim + 255) / 256), dim3(256), 0, st, psum, pcount,
                           static_cast<uint32_t>(small_blocks), dim, k, cent, counts_dev);
        VA_HIP(hipGetLastError());
        return 0;
    }
    uint32_t blocks = static_cast<uint32_t>(div_up(n, 256));
    hipLaunchKernelGGL(fill_u64_kernel, dim3((k / 2 + 1 + 255) / 256), dim3(256), 0, st,
                       reinterpret_cast<unsigned long long*>(b.counts), 0ull, static_cast<uint64_t>(k / 2 + 1));
    hipLaunchKernelGGL(count_labels_kernel, dim3(blocks), dim3(256), 0, st, labels, n, k, b.counts);
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(1024), 0, st, b.counts, k, b.offsets);
    hipLaunchKernelGGL(iota_u32_kernel, dim3(blocks), dim3(256), 0, st, b.rows_in, n);
    int end_bit = 1;
    while ((1ull << end_bit) < k) {
        ++end_bit;
    }
    size_t tmp_bytes = b.sort_tmp_bytes;
    VA_HIP(hipcub::DeviceRadixSort::SortPairs(b.sort_tmp, tmp_bytes, labels, b.keys_out, b.rows_in, b.rows_out,
                                              static_cast<int>(n), 0, end_bit, st));
    hipLaunchKernelGGL(centroid_mean_kernel, dim3(k), dim3(256), 0, st, x, dim, b.rows_out, b.offsets, cent,
                       counts_dev);
    VA_HIP(hipGetLastError());
    return 0;
}

static int
check_kmeans(const void* x, uint64_t n, uint32_t dim, const void* cent, uint32_t k) {
    VA_CHECK_ARG(k >= 1, "k must be positive");
    VA_CHECK_ARG(n >= 1, "count must be positive");
    VA_CHECK_ARG(x != nullptr && cent != nullptr, "datas cannot be null");
    VA_CHECK_ARG(dim >= 1 && dim <= 65536, "dim must be in [1, 65536], got %u", dim);
    VA_CHECK_ARG(n < (1ull << 31), "n must be below 2^31");
    return 0;
}

// ---- k-means++ seeding (KMeansCluster::select_initial_centroids_kmeans_plus_plus, kmeans_cluster.cpp:383-435) -------
// One step = two launches: the distance of every row to the centroid chosen last lowers the row's smallest distance
// so far, and a row is drawn with a probability proportional to that distance -- the first row at which the running
// sum of the distances (a double, in row order) reaches the step's threshold draw * total.  The reference sums
// sequentially; here a block of 64 rows is summed in row order, blocks in chunks in block order, chunks in chunk
// order, chunks in runs: the same sums apart from the association of the double additions.
constexpr uint32_t kPpRows = 64;      // rows per workgroup of the distance launch (one wave, a lane per row)
constexpr uint32_t kPpChunks = 1024;  // threads of the picking workgroup: each sums a run of block sums

__global__ void __launch_bounds__(64)
kpp_distance_kernel(const float* x, uint64_t n, uint32_t dim, const float* centroid, float* min_dist, double* block_sum,
                    int first_step) {
    __shared__ float rows[kPpRows][kPpRows + 1];
    __shared__ float cent[kPpRows];
    __shared__ float md[kPpRows];
    const uint32_t lane = threadIdx.x;
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * kPpRows;
    // FP32ComputeL2Sqr in element order (simd/generic.cpp): result += (a - b) * (a - b), one row per lane.
    float result = 0.0F;
    for (uint32_t c0 = 0; c0 < dim; c0 += kPpRows) {
        const uint32_t d = c0 + lane;
        cent[lane] = d < dim ? centroid[d] : 0.0F;
        // All 64 loads of the chunk are issued before the first is used (no branch around a load: addresses are
        // clamped, what lies beyond the data is never used).
        const uint32_t dc = d < dim ? d : dim - 1;
        float v[kPpRows];
#pragma unroll
        for (uint32_t r = 0; r < kPpRows; ++r) {
            const uint64_t row = row0 + r < n ? row0 + r : n - 1;
            v[r] = x[row * dim + dc];
        }
#pragma unroll
        for (uint32_t r = 0; r < kPpRows; ++r) {
            rows[r][lane] = v[r];
        }
        __syncthreads();
        const uint32_t width = dim - c0 < kPpRows ? dim - c0 : kPpRows;
        for (uint32_t j = 0; j < width; ++j) {
            const float diff = rows[lane][j] - cent[j];
            result += diff * diff;
        }
        __syncthreads();
    }
    const uint64_t row = row0 + lane;
    float m = 0.0F;
    if (row < n) {
        const float old = first_step ? 3.402823466e38F : min_dist[row];
        m = result < old ? result : old;  // std::min(min_distances[i], dist)
        min_dist[row] = m;
    }
    md[lane] = m;
    __syncthreads();
    if (lane == 0) {
        double sum = 0.0;
        for (uint32_t r = 0; r < kPpRows; ++r) {
            sum += static_cast<double>(md[r]);
        }
        block_sum[blockIdx.x] = sum;
    }
}

// One workgroup.  The walk along the running sum goes down four levels -- 32 runs of 32 chunks, the chunks of a run,
// the block sums of a chunk, the 64 rows of a block -- and one thread does each walk over values the others have
// brought into LDS, so that no step of a walk waits for global memory.
__global__ void __launch_bounds__(kPpChunks)
kpp_pick_kernel(const float* x, uint64_t n, uint32_t dim, const float* min_dist, const double* block_sum,
                uint64_t nblocks, double draw, float* centroid_out, uint64_t* pick_out) {
    constexpr uint32_t kRuns = 32, kPerRun = kPpChunks / kRuns;
    __shared__ double chunk_sum[kPpChunks];
    __shared__ double run_sum[kRuns];
    __shared__ double staged[kPpChunks];
    __shared__ double cumulative_s, threshold_s;
    __shared__ uint64_t at_s;  // the chunk, then the block, then the row the walk has reached
    __shared__ int done_s;
    const uint32_t t = threadIdx.x;
    const uint64_t per = (nblocks + kPpChunks - 1) / kPpChunks;
    const uint64_t b0 = t * per, b1 = b0 + per < nblocks ? b0 + per : nblocks;
    double mine = 0.0;
    for (uint64_t b = b0; b < b1; ++b) {
        mine += block_sum[b];
    }
    chunk_sum[t] = mine;
    __syncthreads();
    if (t < kRuns) {
        double r = 0.0;
        for (uint32_t c = 0; c < kPerRun; ++c) {
            r += chunk_sum[t * kPerRun + c];
        }
        run_sum[t] = r;
    }
    __syncthreads();
    if (t == 0) {
        double total = 0.0;
        for (uint32_t r = 0; r < kRuns; ++r) {
            total += run_sum[r];
        }
        done_s = 0;
        if (!(total > 0.0)) {
            // Every row coincides with a centroid: any row (uniform_int_distribution in the reference).
            const double f = draw * static_cast<double>(n);
            at_s = f >= static_cast<double>(n - 1) ? n - 1 : static_cast<uint64_t>(f);
            done_s = 1;
        } else {
            const double threshold = draw * total;
            double cumulative = 0.0;
            uint32_t r = 0;
            while (r + 1 < kRuns && !(cumulative + run_sum[r] >= threshold)) {
                cumulative += run_sum[r];
                ++r;
            }
            uint32_t c = r * kPerRun;
            while (c + 1 < (r + 1) * kPerRun && !(cumulative + chunk_sum[c] >= threshold)) {
                cumulative += chunk_sum[c];
                ++c;
            }
            cumulative_s = cumulative;
            threshold_s = threshold;
            at_s = c;
        }
    }
    __syncthreads();
    if (done_s == 0) {
        // The block sums of the chunk, kPpChunks at a time.
        const uint64_t first = at_s * per;
        const uint64_t last = first + per < nblocks ? first + per : nblocks;  // may be <= first: a chunk without blocks
        __syncthreads();
        if (t == 0) {
            at_s = last > first ? last - 1 : (nblocks - 1);
        }
        for (uint64_t base = first; base < last; base += kPpChunks) {
            if (base + t < last) {
                staged[t] = block_sum[base + t];
            }
            __syncthreads();
            if (t == 0 && done_s == 0) {
                const uint64_t m = last - base < kPpChunks ? last - base : kPpChunks;
                double cumulative = cumulative_s;
                for (uint64_t i = 0; i < m; ++i) {
                    if (base + i + 1 == last || cumulative + staged[i] >= threshold_s) {
                        at_s = base + i;
                        done_s = 2;
                        break;
                    }
                    cumulative += staged[i];
                }
                cumulative_s = cumulative;
            }
            __syncthreads();
            if (done_s != 0) {
                break;
            }
        }
        __syncthreads();
        const uint64_t blk = at_s;
        const uint64_t r0 = blk * kPpRows, r1 = r0 + kPpRows < n ? r0 + kPpRows : n;
        if (t < kPpRows) {
            staged[t] = r0 + t < r1 ? static_cast<double>(min_dist[r0 + t]) : 0.0;
        }
        __syncthreads();
        if (t == 0) {
            uint64_t idx = r1 - 1;
            double cumulative = cumulative_s;
            for (uint64_t r = r0; r < r1; ++r) {
                cumulative += staged[r - r0];
                if (cumulative >= threshold_s) {
                    idx = r;
                    break;
                }
            }
            at_s = idx;
        }
        __syncthreads();
    }
    const uint64_t idx = at_s;
    if (t == 0 && pick_out != nullptr) {
        *pick_out = idx;
    }
    for (uint32_t d = t; d < dim; d += kPpChunks) {
        centroid_out[d] = x[idx * dim + d];
    }
}

}  // namespace vsag_amd

using namespace vsag_amd;

extern "C" size_t
vsag_amd_kmeans_init_plus_plus_workspace_bytes(uint64_t n) {
    Carver c(nullptr, 0);
    c.take<float>(n);
    c.take<double>(div_up(n, static_cast<uint64_t>(kPpRows)));
    return c.used + 256;
}

extern "C" int
vsag_amd_kmeans_init_plus_plus(const float* x_dev, uint64_t n, uint32_t dim, uint32_t k, uint64_t first,
                               const double* draws, float* centroids_dev, uint64_t* picks_dev, void* workspace_dev,
                               size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_kmeans(x_dev, n, dim, centroids_dev, k));
    VA_CHECK_ARG(k <= n, "k cannot be larger than count");
    VA_CHECK_ARG(first < n, "the first centroid must be a row of the data");
    VA_CHECK_ARG(k == 1 || draws != nullptr, "draws is null");
    for (uint32_t c = 1; c < k; ++c) {
        VA_CHECK_ARG(draws[c - 1] >= 0.0 && draws[c - 1] < 1.0, "draws must lie in [0, 1)");
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver c(workspace_dev, workspace_bytes);
    float* min_dist = c.take<float>(n);
    const uint64_t nblocks = div_up(n, static_cast<uint64_t>(kPpRows));
    double* block_sum = c.take<double>(nblocks);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    VA_HIP(hipMemcpyAsync(centroids_dev, x_dev + first * dim, dim * sizeof(float), hipMemcpyDeviceToDevice, st));
    if (picks_dev != nullptr) {
        VA_HIP(hipMemcpyAsync(picks_dev, &first, sizeof(uint64_t), hipMemcpyHostToDevice, st));
        VA_HIP(hipStreamSynchronize(st));  // `first` lives on this frame
    }
    for (uint32_t j = 1; j < k; ++j) {
        hipLaunchKernelGGL(kpp_distance_kernel, dim3(static_cast<uint32_t>(nblocks)), dim3(kPpRows), 0, st, x_dev, n, dim,
                           centroids_dev + static_cast<uint64_t>(j - 1) * dim, min_dist, block_sum, j == 1 ? 1 : 0);
        hipLaunchKernelGGL(kpp_pick_kernel, dim3(1), dim3(kPpChunks), 0, st, x_dev, n, dim, min_dist, block_sum, nblocks,
                           draws[j - 1], centroids_dev + static_cast<uint64_t>(j) * dim,
                           picks_dev != nullptr ? picks_dev + j : nullptr);
    }
    VA_HIP(hipGetLastError());
    return 0;
}

extern "C" size_t
vsag_amd_kmeans_assign_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k) {
    (void)dim;
    Carver c(nullptr, 0);
    AssignBuffers b;
    return carve_assign(c, n, k, &b) + 256;
}

extern "C" int
vsag_amd_kmeans_assign(const float* x_dev, uint64_t n, uint32_t dim, const float* centroids_dev, uint32_t k,
                       int32_t* labels_dev, float* min_dist_dev, double* loss_dev, void* workspace_dev,
                       size_t workspace_bytes, void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_kmeans(x_dev, n, dim, centroids_dev, k));
    VA_CHECK_ARG(labels_dev != nullptr, "labels_dev is null");
    Carver c(workspace_dev, workspace_bytes);
    AssignBuffers b;
    carve_assign(c, n, k, &b);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    return assign_launch(x_dev, n, dim, centroids_dev, k, labels_dev, min_dist_dev, loss_dev, b, false,
                         static_cast<hipStream_t>(stream));
}

extern "C" size_t
vsag_amd_kmeans_update_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k) {
    (void)dim;
    if (ensure_init() != 0) {
        return 0;
    }
    Carver c(nullptr, 0);
    UpdateBuffers b;
    return carve_update(c, n, k, &b) + 256;
}

extern "C" int
vsag_amd_kmeans_update(const float* x_dev, const int32_t* labels_dev, uint64_t n, uint32_t dim, uint32_t k,
                       float* centroids_dev, int32_t* counts_dev, void* workspace_dev, size_t workspace_bytes,
                       void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_kmeans(x_dev, n, dim, centroids_dev, k));
    VA_CHECK_ARG(labels_dev != nullptr && counts_dev != nullptr, "null labels / counts");
    Carver c(workspace_dev, workspace_bytes);
    UpdateBuffers b;
    carve_update(c, n, k, &b);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);
    return update_launch(x_dev, labels_dev, n, dim, k, centroids_dev, counts_dev, b, static_cast<hipStream_t>(stream));
}

extern "C" size_t
vsag_amd_kmeans_run_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k) {
    (void)dim;
    if (ensure_init() != 0) {
        return 0;
    }
    Carver c(nullptr, 0);
    AssignBuffers a;
    UpdateBuffers u;
    carve_assign(c, n, k, &a);
    carve_update(c, n, k, &u);
    c.take<int32_t>(k);
    return c.used + 256;
}

extern "C" int
vsag_amd_kmeans_run(const float* x_dev, uint64_t n, uint32_t dim, float* centroids_dev, uint32_t k, int iters,
                    uint64_t seed, int32_t* labels_dev, double* loss, void* workspace_dev, size_t workspace_bytes,
                    void* stream) {
    VA_TRY(ensure_init());
    VA_TRY(check_kmeans(x_dev, n, dim, centroids_dev, k));
    VA_CHECK_ARG(k <= n, "k cannot be larger than count");
    VA_CHECK_ARG(labels_dev != nullptr, "labels_dev is null");
    VA_CHECK_ARG(iters >= 0, "iters must not be negative");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver c(workspace_dev, workspace_bytes);
    AssignBuffers a;
    UpdateBuffers u;
    carve_assign(c, n, k, &a);
    carve_update(c, n, k, &u);
    int32_t* counts_dev = c.take<int32_t>(k);
    VA_CHECK_ARG(c.ok(), "workspace too small: need %zu bytes, got %zu", c.used, workspace_bytes);

    std::mt19937 gen(static_cast<uint32_t>(seed));
    std::vector<int32_t> counts(k);
    double last = 0.0;
    for (int it = 0; it < iters; ++it) {
        VA_TRY(assign_launch(x_dev, n, dim, centroids_dev, k, labels_dev, nullptr, a.loss_tmp, a, it > 0, st));
        VA_TRY(update_launch(x_dev, labels_dev, n, dim, k, centroids_dev, counts_dev, u, st));
        VA_HIP(hipMemcpyAsync(counts.data(), counts_dev, k * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        VA_HIP(hipMemcpyAsync(&last, a.loss_tmp, sizeof(double), hipMemcpyDeviceToHost, st));
        VA_HIP(hipStreamSynchronize(st));
        // Empty clusters restart from a random data row (kmeans_cluster.cpp:156-171).
        std::uniform_int_distribution<uint64_t> dis(0, n - 1);
        for (uint32_t j = 0; j < k; ++j) {
            if (counts[j] == 0) {
                uint64_t idx = dis(gen);
                VA_HIP(hipMemcpyAsync(centroids_dev + static_cast<uint64_t>(j) * dim, x_dev + idx * dim,
                                      dim * sizeof(float), hipMemcpyDeviceToDevice, st));
            }
        }
    }
    VA_HIP(hipStreamSynchronize(st));
    if (loss != nullptr) {
        *loss = last;
    }
    return 0;
}
