// RMSNorm forward / backward for gfx950 (math: cute_kernels/kernels/rmsnorm/README.md:3-25).
//
// Fast path (row length a multiple of the 16-byte packet, 16-byte aligned pointers):
//   a "team" of TPR lanes (64, 256 or 1024) owns one row at a time and keeps it in registers, so x (and
//   dy) are read from HBM exactly once.  Row sums use wave64 shuffles; teams wider than a wave finish
//   through a few LDS floats.  Backward is persistent: each team walks rows team, team+teams, ... and
//   accumulates its share of dweight in fp32 registers; the teams of a workgroup add their shares up through
//   LDS and write one fp32 partial row per workgroup to the workspace, and a second kernel sums the partial
//   rows column-wise with shuffles.  No atomics anywhere, so dweight is deterministic for a given team count.
// Generic path (any H, any element alignment): one 256-lane team per row re-reading the row from cache,
//   and a column kernel for the dweight partials.
#include <map>
#include <mutex>

#include "ck_device.h"

namespace ck {

constexpr int kMaxPacks = 8;        // packets a lane keeps per row on the fast path
constexpr int kColSegments = 64;    // row segments of the generic dweight column kernel

// sum over the TPR lanes that share a row; `red` is LDS scratch of (blockDim/64) floats per use
template <int TPR>
__device__ __forceinline__ float team_sum(float v, float* red) {
    v = wave_sum(v);
    if (TPR > CK_WAVE) {
        const int wave = threadIdx.x / CK_WAVE;
        __syncthreads();  // protect `red` from the previous use
        if (lane_id() == 0) red[wave] = v;
        __syncthreads();
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < TPR / CK_WAVE; ++w) t += red[w];
        v = t;
    }
    return v;
}

// Registers: the row stays packed in its storage type (8 packets = 32 VGPRs for a 16-bit row of 4096) and is
// widened to fp32 element by element where it is used; the bound of two waves per SIMD keeps the compiler from
// hoisting the widened copies (which would leave one wave per SIMD and nothing to hide latency with).
// Makes the compiler forget what it knows about a packed register set: values widened from it before this
// point cannot be kept alive in place of the packed form.
template <typename P>
__device__ __forceinline__ void forget(P& p) {
    static_assert(sizeof(P) % 4 == 0, "whole registers");
    uint32_t* w = reinterpret_cast<uint32_t*>(&p);
#pragma unroll
    for (int i = 0; i < (int)(sizeof(P) / 4); ++i) asm volatile("" : "+v"(w[i]));
}

#define CK_RMS_BOUNDS(TPR) __launch_bounds__((TPR) > 256 ? (TPR) : 256, (TPR) > 256 ? 1 : 2)

// RES: the row that is normalised is x + res, rounded to the storage type and written to res_out as well (the
// residual stream of a transformer block: one pass instead of an addition followed by a normalisation).
// NP: packets per lane when the row is exactly NP * TPR packets long (no lane ever idles, so no packet sits behind a
// branch and the loads of a row are issued back to back); 0: any row length, every packet predicated.
template <typename T, int TPR, bool RES = false, int NP = 0>
__global__ void CK_RMS_BOUNDS(TPR)
    rmsnorm_fwd_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                       typename T::storage_t* __restrict__ y, float* __restrict__ rstd_out, int64_t B, int H,
                       float eps, const typename T::storage_t* __restrict__ res = nullptr,
                       typename T::storage_t* __restrict__ res_out = nullptr) {
    typedef VPack<T, T::kVec> P;
    constexpr int N = NP != 0 ? NP : kMaxPacks;
    __shared__ float red[16];
    const int teams_per_block = blockDim.x / TPR;
    const int team = blockIdx.x * teams_per_block + threadIdx.x / TPR;
    const int num_teams = gridDim.x * teams_per_block;
    const int t = threadIdx.x % TPR;
    const int packs = H / T::kVec;
    const float inv_h = 1.0f / (float)H;

    // rows are dealt round-robin; the next row is requested before the current one is reduced.
    // With TPR > 64 the block is one team, so the trip count is uniform across the barriers in team_sum.
    P cur[kMaxPacks], nxt[kMaxPacks];
    P rcur[RES ? kMaxPacks : 1], rnxt[RES ? kMaxPacks : 1];
    // the weight stays in registers (packed) for all rows of the team: fetched per row it is as many requests to
    // the L1 / L2 path as the row itself (measured: 55 instead of 49 us at 16384 rows of 4096)
    // (where the registers allow: the 1024-lane team has 128 per lane, and the 256-lane team with a residual needs them)
    constexpr bool HOIST_W = TPR == 64 || (TPR == 256 && !RES);
    P wreg[HOIST_W ? kMaxPacks : 1];
    if (HOIST_W && w != nullptr) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) wreg[i] = reinterpret_cast<const P*>(w)[p];
        }
    }
    int64_t row = team;
    if (row < B) {
        const P* xr = reinterpret_cast<const P*>(x + row * H);
        const P* rr = RES ? reinterpret_cast<const P*>(res + row * H) : nullptr;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
                cur[i] = nt_load(xr + p);
                if (RES) rcur[i] = nt_load(rr + p);
            }
        }
    }
    for (; row < B; row += num_teams) {
        const int64_t next_row = row + num_teams;
        if (next_row < B) {
            const P* xr = reinterpret_cast<const P*>(x + next_row * H);
            const P* rr = RES ? reinterpret_cast<const P*>(res + next_row * H) : nullptr;
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = t + i * TPR;
                if (NP != 0 || p < packs) {
                    nxt[i] = nt_load(xr + p);
                    if (RES) rnxt[i] = nt_load(rr + p);
                }
            }
        }
        if (RES) {
            // the sum is rounded to the storage type first: that value is both the new residual and the row that
            // is normalised, exactly as an addition kernel followed by the normalisation would have it
            P* so = reinterpret_cast<P*>(res_out + row * H);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = t + i * TPR;
                if (NP != 0 || p < packs) {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) cur[i].v[j] = T::down(T::up(cur[i].v[j]) + T::up(rcur[i].v[j]));
                    nt_store(cur[i], so + p);
                }
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
#pragma unroll
                for (int j = 0; j < T::kVec; ++j) {
                    const float f = T::up(cur[i].v[j]);
                    ss += f * f;
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one packet at a time: the widened values do not pile up
        }
        if (sizeof(typename T::storage_t) == 2) {
            // 16-bit rows: only the packed form lives across the reduction (the widened copies would double the
            // registers and halve the waves per SIMD)
#pragma unroll
            for (int i = 0; i < N; ++i) {
                forget(cur[i]);
                if (HOIST_W) forget(wreg[i]);
            }
        }
        ss = team_sum<TPR>(ss, red);
        const float rstd = rsqrtf(ss * inv_h + eps);
        if (rstd_out != nullptr && t == 0) rstd_out[row] = rstd;

        P* yr = reinterpret_cast<P*>(y + row * H);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
                P o;
                if (w != nullptr) {
                    const P wv = HOIST_W ? wreg[HOIST_W ? i : 0] : reinterpret_cast<const P*>(w)[p];
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) o.v[j] = T::down(T::up(cur[i].v[j]) * rstd * T::up(wv.v[j]));
                } else {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) o.v[j] = T::down(T::up(cur[i].v[j]) * rstd);
                }
                nt_store(o, yr + p);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < N; ++i) {
            cur[i] = nxt[i];
            if (RES) rcur[i] = rnxt[i];
        }
    }
}

// Rows of up to 64 * kMaxPacks packets, forward, without the walk over rows: one wave takes RPW consecutive rows,
// requests all of them at once, reduces and writes them, and ends.  Few registers (the rows in their packed form), so
// many waves per SIMD are resident and their requests overlap each other's reductions - the persistent kernel above
// holds two rows per wave in 134 registers, three waves per SIMD, and its fourth workgroup per compute unit only
// starts when another has ended.  RPW > 1 reads the weight once for RPW rows.
template <typename T, int RPW, bool RES = false, int NP = 0>
__global__ void __launch_bounds__(256)
    rmsnorm_fwd_rows_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                            typename T::storage_t* __restrict__ y, float* __restrict__ rstd_out, int64_t B, int H,
                            float eps, const typename T::storage_t* __restrict__ res = nullptr,
                            typename T::storage_t* __restrict__ res_out = nullptr) {
    typedef VPack<T, T::kVec> P;
    constexpr int N = NP != 0 ? NP : kMaxPacks;
    const int lane = lane_id();
    const int packs = H / T::kVec;
    const float inv_h = 1.0f / (float)H;
    const int64_t row0 = ((int64_t)blockIdx.x * (blockDim.x / CK_WAVE) + threadIdx.x / CK_WAVE) * RPW;
    if (row0 >= B) return;
    P v[RPW][kMaxPacks], r[RES ? RPW : 1][RES ? kMaxPacks : 1];
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        if (row0 + q < B) {
            const P* xr = reinterpret_cast<const P*>(x + (row0 + q) * H);
            const P* rr = RES ? reinterpret_cast<const P*>(res + (row0 + q) * H) : nullptr;
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = lane + i * CK_WAVE;
                if (NP != 0 || p < packs) {
                    v[q][i] = nt_load(xr + p);
                    if (RES) r[q][i] = nt_load(rr + p);
                }
            }
        }
    }
    P wv[kMaxPacks];
    if (w != nullptr) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = lane + i * CK_WAVE;
            if (NP != 0 || p < packs) wv[i] = reinterpret_cast<const P*>(w)[p];
        }
    }
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        const int64_t row = row0 + q;
        if (row >= B) break;
        if (RES) {
            // the sum is rounded to the storage type first: that value is both the new residual and the row that is
            // normalised, exactly as an addition kernel followed by the normalisation would have it
            P* so = reinterpret_cast<P*>(res_out + row * H);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = lane + i * CK_WAVE;
                if (NP != 0 || p < packs) {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) v[q][i].v[j] = T::down(T::up(v[q][i].v[j]) + T::up(r[q][i].v[j]));
                    nt_store(v[q][i], so + p);
                }
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = lane + i * CK_WAVE;
            if (NP != 0 || p < packs) {
#pragma unroll
                for (int j = 0; j < T::kVec; ++j) {
                    const float f = T::up(v[q][i].v[j]);
                    ss += f * f;
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one packet at a time: the widened values do not pile up
        }
        if (sizeof(typename T::storage_t) == 2) {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                forget(v[q][i]);
                forget(wv[i]);
            }
        }
        ss = wave_sum(ss);
        const float rstd = rsqrtf(ss * inv_h + eps);
        if (rstd_out != nullptr && lane == 0) rstd_out[row] = rstd;
        P* yr = reinterpret_cast<P*>(y + row * H);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = lane + i * CK_WAVE;
            if (NP != 0 || p < packs) {
                P o;
                if (w != nullptr) {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) o.v[j] = T::down(T::up(v[q][i].v[j]) * rstd * T::up(wv[i].v[j]));
                } else {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) o.v[j] = T::down(T::up(v[q][i].v[j]) * rstd);
                }
                nt_store(o, yr + p);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Backward: one wave per SIMD with the whole register file (packed current row and next row of x and dy, packed
// weight, 64 fp32 dweight accumulators); the next row's loads are in flight while the current row is reduced.
// NEED_SS = false: 1 / rms is given, and the row's sum of squares - one multiply-add per element and a reduction over
// the team - is not computed at all (5 us of 81 at 16384 x 4096).  NEED_SS = true forms it unless rstd_in is given
// (the 1024-lane team is compiled this way only: without the sum its register allocation spills).
template <typename T, int TPR, bool HAS_W, bool PREFETCH, int NP, bool NEED_SS>
__device__ __forceinline__ void rmsnorm_bwd_body(const typename T::storage_t* __restrict__ x,
                                                 const typename T::storage_t* __restrict__ w,
                                                 const typename T::storage_t* __restrict__ dy,
                                                 const float* __restrict__ rstd_in, typename T::storage_t* __restrict__ dx,
                                                 float* __restrict__ dw_partial, int64_t B, int H, float eps) {
    typedef VPack<T, T::kVec> P;
    constexpr int N = NP != 0 ? NP : kMaxPacks;
    // The 1024-lane team has 128 registers per lane.  With a weight, the packed x, dy and weight of the row plus the
    // 64 fp32 dweight accumulators are 160: the compiler then spills 500 bytes per lane and the kernel runs seven
    // times longer than without a weight (538 against 75 us at 2048 x 32768).  So there only the accumulators are
    // kept: x, dy and the weight are read twice, the second time from the cache the first read left them in.
    constexpr bool LEAN = HAS_W && TPR == 1024;
    __shared__ float red[16];
    const int teams_per_block = blockDim.x / TPR;
    const int team = blockIdx.x * teams_per_block + threadIdx.x / TPR;
    const int num_teams = gridDim.x * teams_per_block;
    const int t = threadIdx.x % TPR;
    const int packs = H / T::kVec;
    const float inv_h = 1.0f / (float)H;

    P wv[LEAN ? 1 : kMaxPacks];
    float dw[kMaxPacks][T::kVec];
    if (HAS_W) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (!LEAN && (NP != 0 || p < packs)) wv[i] = reinterpret_cast<const P*>(w)[p];
#pragma unroll
            for (int j = 0; j < T::kVec; ++j) dw[i][j] = 0.f;
        }
    }

    // rows are dealt round-robin; with TPR > 64 the block is one team so the trip count is block-uniform
    static_assert(!(LEAN && PREFETCH), "the lean form has no row in flight");
    P xv[LEAN ? 1 : kMaxPacks], gv[LEAN ? 1 : kMaxPacks], xn[PREFETCH ? kMaxPacks : 1], gn[PREFETCH ? kMaxPacks : 1];
    if (PREFETCH && team < B) {
        const P* xr = reinterpret_cast<const P*>(x + (int64_t)team * H);
        const P* gr = reinterpret_cast<const P*>(dy + (int64_t)team * H);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
                xv[i] = nt_load(xr + p);
                gv[i] = nt_load(gr + p);
            }
        }
    }
    for (int64_t row = team; row < B; row += num_teams) {
        // 1/rms of this row, requested BEFORE the next row's packets: loads complete in the order they were issued,
        // so a value requested behind them would not arrive before they all have - the wait for it would be a wait
        // for the whole row that is meant to stay in flight during this row's arithmetic
        float rstd_given = 0.f;
        if (!NEED_SS || rstd_in != nullptr) rstd_given = rstd_in[row];
        if (PREFETCH) {
            const int64_t next_row = row + num_teams;
            if (next_row < B) {
                const P* xr = reinterpret_cast<const P*>(x + next_row * H);
                const P* gr = reinterpret_cast<const P*>(dy + next_row * H);
#pragma unroll
                for (int i = 0; i < N; ++i) {
                    const int p = t + i * TPR;
                    if (NP != 0 || p < packs) {
                        xn[i] = nt_load(xr + p);
                        gn[i] = nt_load(gr + p);
                    }
                }
            }
        } else if (!LEAN) {
            const P* xr = reinterpret_cast<const P*>(x + row * H);
            const P* gr = reinterpret_cast<const P*>(dy + row * H);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = t + i * TPR;
                if (NP != 0 || p < packs) {
                    xv[i] = nt_load(xr + p);
                    gv[i] = nt_load(gr + p);
                }
            }
        }
        float ss = 0.f, dot = 0.f;
        if (LEAN) {
            // everything passes through (plain loads: the packets are wanted again below), two packets at a time
            const P* xr = reinterpret_cast<const P*>(x + row * H);
            const P* gr = reinterpret_cast<const P*>(dy + row * H);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = t + i * TPR;
                if (NP != 0 || p < packs) {
                    const P x8 = xr[p];
                    const P g8 = gr[p];
                    const P w8 = reinterpret_cast<const P*>(w)[p];
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) {
                        const float xf = T::up(x8.v[j]);
                        if (NEED_SS) ss += xf * xf;
                        dot += T::up(g8.v[j]) * T::up(w8.v[j]) * xf;
                    }
                }
                if (i % 2 == 1) __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const int p = t + i * TPR;
                if (NP != 0 || p < packs) {
#pragma unroll
                    for (int j = 0; j < T::kVec; ++j) {
                        const float xf = T::up(xv[i].v[j]);
                        float g = T::up(gv[i].v[j]);
                        if (HAS_W) g *= T::up(wv[i].v[j]);
                        if (NEED_SS) ss += xf * xf;
                        dot += g * xf;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (!LEAN && sizeof(typename T::storage_t) == 2) {
            // 16-bit rows: keep only the packed form across the reductions
#pragma unroll
            for (int i = 0; i < N; ++i) {
                forget(xv[i]);
                forget(gv[i]);
                if (HAS_W) forget(wv[i]);
            }
        }
        float rstd;
        if (!NEED_SS || rstd_in != nullptr) {
            rstd = rstd_given;
        } else {
            ss = team_sum<TPR>(ss, red);
            rstd = rsqrtf(ss * inv_h + eps);
        }
        dot = team_sum<TPR>(dot, red);
        const float c = rstd * rstd * rstd * inv_h * dot;

        P* dr = reinterpret_cast<P*>(dx + row * H);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
                P o;
                P x8, g8, w8;
                if (LEAN) {
                    x8 = reinterpret_cast<const P*>(x + row * H)[p];
                    g8 = reinterpret_cast<const P*>(dy + row * H)[p];
                    w8 = reinterpret_cast<const P*>(w)[p];
                } else {
                    x8 = xv[LEAN ? 0 : i];
                    g8 = gv[LEAN ? 0 : i];
                    if (HAS_W) w8 = wv[LEAN ? 0 : i];
                }
#pragma unroll
                for (int j = 0; j < T::kVec; ++j) {
                    const float xf = T::up(x8.v[j]);
                    const float d = T::up(g8.v[j]);
                    float g = d;
                    if (HAS_W) {
                        g *= T::up(w8.v[j]);
                        dw[i][j] += d * (xf * rstd);
                    }
                    o.v[j] = T::down(rstd * g - c * xf);
                }
                nt_store(o, dr + p);
            }
            // one packet at a time: keeps the widened values of later packets from piling up in registers
            __builtin_amdgcn_sched_barrier(0);
        }
        if (PREFETCH) {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                xv[i] = xn[i];
                gv[i] = gn[i];
            }
        }
    }

    if (HAS_W) {
        // One partial row per workgroup.  With one wave per row a workgroup holds four teams: their rows are added
        // up through LDS first (in team order), which quarters what the reduce pass has to read.
        constexpr int kTeams = TPR == 64 ? 4 : 1;
        constexpr int kCols = TPR == 64 ? 64 * kMaxPacks * T::kVec : 4;
        __shared__ float comb[kTeams > 1 ? kTeams * kCols : 4];
        float* out = kTeams > 1 ? comb + (threadIdx.x / TPR) * kCols : dw_partial + (int64_t)team * H;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = t + i * TPR;
            if (NP != 0 || p < packs) {
#pragma unroll
                for (int j = 0; j < T::kVec; j += 4) {
                    float4 v = make_float4(dw[i][j], dw[i][j + 1], dw[i][j + 2], dw[i][j + 3]);
                    *reinterpret_cast<float4*>(out + p * T::kVec + j) = v;
                }
            }
        }
        if (kTeams > 1) {
            __syncthreads();
            float* row = dw_partial + (int64_t)blockIdx.x * H;
            for (int c = threadIdx.x * 4; c < H; c += blockDim.x * 4) {
                float4 a = *reinterpret_cast<const float4*>(comb + c);
#pragma unroll
                for (int k = 1; k < kTeams; ++k) {
                    const float4 b = *reinterpret_cast<const float4*>(comb + k * kCols + c);
                    a.x += b.x;
                    a.y += b.y;
                    a.z += b.z;
                    a.w += b.w;
                }
                *reinterpret_cast<float4*>(row + c) = a;
            }
        }
    }
}

// The next row of x and dy in flight while the current one is reduced: 288 registers with a weight at a row length
// of 4096, i.e. one wave per SIMD and one workgroup per compute unit (the 1024-lane variant has 128 registers per
// lane and no room for it).
template <typename T, int TPR, bool HAS_W, int NP, bool NEED_SS>
__global__ void __launch_bounds__(TPR > 256 ? TPR : 256)
    rmsnorm_bwd_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                       const typename T::storage_t* __restrict__ dy, const float* __restrict__ rstd_in,
                       typename T::storage_t* __restrict__ dx, float* __restrict__ dw_partial, int64_t B, int H,
                       float eps) {
    rmsnorm_bwd_body<T, TPR, HAS_W, TPR <= 256, NP, NEED_SS>(x, w, dy, rstd_in, dx, dw_partial, B, H, eps);
}

// One wave per row without the row in flight: fits two waves per SIMD, so two workgroups per compute unit walk the
// rows and one wave's loads overlap the other's reductions and stores.
template <typename T, bool HAS_W, int NP, bool NEED_SS>
__global__ void __launch_bounds__(256, 2)
    rmsnorm_bwd_two_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                           const typename T::storage_t* __restrict__ dy, const float* __restrict__ rstd_in,
                           typename T::storage_t* __restrict__ dx, float* __restrict__ dw_partial, int64_t B, int H,
                           float eps) {
    rmsnorm_bwd_body<T, 64, HAS_W, false, NP, NEED_SS>(x, w, dy, rstd_in, dx, dw_partial, B, H, eps);
}

// dweight[j] = sum over `parts` partial rows of partial[r][j].  One wave per block owns 16 columns:
// lane = 16 row-groups x 4 column-quads; each lane strides over the partial rows with float4 loads,
// then the 16 row-groups are folded with shuffles.  Requires H % 4 == 0.
// With gridDim.y > 1 the partial rows are split over blockIdx.y and the result goes, still in fp32, to
// `out32` ([gridDim.y][H]); a second launch with gridDim.y == 1 then folds those rows into `dw`.
template <typename T>
__global__ void __launch_bounds__(64)
    rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, typename T::storage_t* __restrict__ dw,
                             float* __restrict__ out32, int parts, int H) {
    const int lane = threadIdx.x;
    const int quad = lane & 3;
    const int group = lane >> 2;
    const int col = blockIdx.x * 16 + quad * 4;
    const int per_split = (parts + gridDim.y - 1) / gridDim.y;
    const int r0 = blockIdx.y * per_split;
    const int r1 = min(r0 + per_split, parts);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (col < H) {
        for (int r = r0 + group; r < r1; r += 16) {
            const float4 v = *reinterpret_cast<const float4*>(partial + (int64_t)r * H + col);
            acc.x += v.x;
            acc.y += v.y;
            acc.z += v.z;
            acc.w += v.w;
        }
    }
#pragma unroll
    for (int off = 4; off < CK_WAVE; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off, CK_WAVE);
        acc.y += __shfl_xor(acc.y, off, CK_WAVE);
        acc.z += __shfl_xor(acc.z, off, CK_WAVE);
        acc.w += __shfl_xor(acc.w, off, CK_WAVE);
    }
    if (group == 0 && col < H) {
        if (out32 != nullptr) {
            *reinterpret_cast<float4*>(out32 + (int64_t)blockIdx.y * H + col) = acc;
        } else {
            dw[col + 0] = T::down(acc.x);
            dw[col + 1] = T::down(acc.y);
            dw[col + 2] = T::down(acc.z);
            dw[col + 3] = T::down(acc.w);
        }
    }
}

// ---- generic path ---------------------------------------------------------------------------
__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if (lane_id() == 0) red[threadIdx.x / CK_WAVE] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

template <typename T>
__global__ void __launch_bounds__(256)
    rmsnorm_fwd_generic_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                               typename T::storage_t* __restrict__ y, float* __restrict__ rstd_out, int64_t B, int H,
                               float eps) {
    __shared__ float red[4];
    for (int64_t row = blockIdx.x; row < B; row += gridDim.x) {
        const typename T::storage_t* xr = x + row * H;
        float ss = 0.f;
        for (int j = threadIdx.x; j < H; j += 256) {
            const float f = T::up(xr[j]);
            ss += f * f;
        }
        ss = block_sum_256(ss, red);
        const float rstd = rsqrtf(ss / (float)H + eps);
        if (rstd_out != nullptr && threadIdx.x == 0) rstd_out[row] = rstd;
        for (int j = threadIdx.x; j < H; j += 256) {
            float v = T::up(xr[j]) * rstd;
            if (w != nullptr) v *= T::up(w[j]);
            y[row * H + j] = T::down(v);
        }
    }
}

// dx for one row per block; also leaves rstd of every row in `rstd_ws` for the column kernel
template <typename T>
__global__ void __launch_bounds__(256)
    rmsnorm_bwd_generic_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ w,
                               const typename T::storage_t* __restrict__ dy, const float* __restrict__ rstd_in,
                               typename T::storage_t* __restrict__ dx, float* __restrict__ rstd_ws, int64_t B, int H,
                               float eps) {
    __shared__ float red[4];
    const float inv_h = 1.0f / (float)H;
    for (int64_t row = blockIdx.x; row < B; row += gridDim.x) {
        const typename T::storage_t* xr = x + row * H;
        const typename T::storage_t* gr = dy + row * H;
        float ss = 0.f, dot = 0.f;
        for (int j = threadIdx.x; j < H; j += 256) {
            const float xf = T::up(xr[j]);
            float g = T::up(gr[j]);
            if (w != nullptr) g *= T::up(w[j]);
            ss += xf * xf;
            dot += g * xf;
        }
        float rstd;
        if (rstd_in != nullptr) {
            rstd = rstd_in[row];
        } else {
            ss = block_sum_256(ss, red);
            rstd = rsqrtf(ss * inv_h + eps);
        }
        dot = block_sum_256(dot, red);
        if (rstd_ws != nullptr && threadIdx.x == 0) rstd_ws[row] = rstd;
        const float c = rstd * rstd * rstd * inv_h * dot;
        for (int j = threadIdx.x; j < H; j += 256) {
            const float xf = T::up(xr[j]);
            float g = T::up(gr[j]);
            if (w != nullptr) g *= T::up(w[j]);
            dx[row * H + j] = T::down(rstd * g - c * xf);
        }
    }
}

// partial[seg][j] = sum over the rows of segment `seg` of dy[b][j] * x[b][j] * rstd[b]; lane per column
template <typename T>
__global__ void __launch_bounds__(256)
    rmsnorm_dw_columns_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ dy,
                              const float* __restrict__ rstd, float* __restrict__ partial, int64_t B, int H,
                              int H_padded) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    const int seg = blockIdx.y;
    const int64_t rows_per_seg = (B + kColSegments - 1) / kColSegments;
    const int64_t b0 = seg * rows_per_seg;
    const int64_t b1 = (b0 + rows_per_seg < B) ? b0 + rows_per_seg : B;
    if (j >= H_padded) return;
    float acc = 0.f;
    if (j < H)
        for (int64_t b = b0; b < b1; ++b) acc += T::up(dy[b * H + j]) * (T::up(x[b * H + j]) * rstd[b]);
    partial[(int64_t)seg * H_padded + j] = acc;
}

template <typename T>
__global__ void __launch_bounds__(256)
    rmsnorm_dw_reduce_generic_kernel(const float* __restrict__ partial, typename T::storage_t* __restrict__ dw,
                                     int parts, int H, int H_padded) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= H) return;
    float acc = 0.f;
    for (int r = 0; r < parts; ++r) acc += partial[(int64_t)r * H_padded + j];
    dw[j] = T::down(acc);
}

}  // namespace ck

// ---- host side ------------------------------------------------------------------------------
constexpr int kReduceSplits = 16;  // row splits of the first dweight reduction pass

static int cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// Workgroups of `kernel` that one compute unit holds at once (registers, LDS): a persistent launch with more than
// that leaves the surplus waiting for a slot while the others already finish their rows.  Looked up once per kernel.
static int resident_blocks(const void* kernel, int block) {
    static std::mutex mutex;
    static std::map<const void*, int> known;
    std::lock_guard<std::mutex> lock(mutex);
    auto it = known.find(kernel);
    if (it != known.end()) return it->second;
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, block, 0) != hipSuccess || n < 1) n = 1;
    if (n > 8) n = 8;
    known[kernel] = n;
    return n;
}

// threads per row on the fast path, 0 when the row does not fit the register budget
static int fast_tpr(int64_t H, int dtype) {
    const int vec = dtype == CK_F32 ? 4 : 8;
    if (H % vec != 0) return 0;
    const int64_t packs = H / vec;
    if (packs <= 64 * ck::kMaxPacks) return 64;
    if (packs <= 256 * ck::kMaxPacks) return 256;
    if (packs <= 1024 * ck::kMaxPacks) return 1024;
    return 0;
}

// teams of the persistent backward kernel (an upper bound of the number of fp32 partial rows)
static int bwd_teams(int64_t B, int tpr, int per_cu = 1) {
    const int block = tpr > 256 ? tpr : 256;
    const int teams_per_block = block / tpr;
    int64_t blocks = (int64_t)cu_count() * per_cu;  // per_cu = 1: the kernel uses the whole register file
    const int64_t need = ck_ceil_div(B, teams_per_block);
    if (blocks > need) blocks = need;
    if (blocks < 1) blocks = 1;
    return (int)(blocks * teams_per_block);
}

// Launch variants of the one-wave-per-row kernels, selected by `block_size_b` (the reference's BLOCK_SIZE_B: rows per
// program): forward 1, 2, 4 = rows a wave requests at once and then ends (rmsnorm_fwd_rows_kernel), 8 or more = waves
// that walk rows with the next one in flight (rmsnorm_fwd_kernel); backward 1 = two workgroups per compute unit
// without a row in flight, 2 or more = one with.  0 = the default.  Rows wider than a wave's registers have one variant.
// The defaults follow what the tuner measured on MI355X at 16384 rows, all three dtypes: rows of up to 2 KB are
// fastest walked (10.9 against 18.4 us at 1024 bf16 elements), longer ones with one wave per row (43.1 against 45.7 us
// at 4096); the backward runs two workgroups per compute unit up to 4 KB a row (22.5 against 27.7 us at 1024, 32.1
// against 33.2 at 2048) and one with a row in flight beyond (66.1 against 71.4 us at 4096).
static int fwd_default_rows(int64_t H, int dtype) { return H * (dtype == CK_F32 ? 4 : 2) <= 2048 ? 8 : 1; }
static int bwd_default_variant(int64_t H, int dtype) { return H * (dtype == CK_F32 ? 4 : 2) <= 4096 ? 1 : 2; }

// packets per lane when a row is exactly that many packets per lane of a TPR-lane team (2, 4 or 8), else 0
static int exact_packs(int64_t H, int dtype, int tpr) {
    const int vec = dtype == CK_F32 ? 4 : 8;
    const int64_t packs = H / vec;
    for (int np : {8, 4, 2})
        if (packs == (int64_t)np * tpr) return np;
    return 0;
}

struct FwdArgs {
    const void *x, *residual, *weight;
    void *output, *residual_out;
    float* rstd;
    int64_t B;
    int H;
    float eps;
};

template <typename T, int RPW, bool RES, int NP>
static void launch_fwd_rows_np(hipStream_t s, const FwdArgs& a) {
    typedef typename T::storage_t S;
    const int64_t grid = ck_ceil_div(a.B, 4 * RPW);
    hipLaunchKernelGGL((ck::rmsnorm_fwd_rows_kernel<T, RPW, RES, NP>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)a.x,
                       (const S*)a.weight, (S*)a.output, a.rstd, a.B, a.H, a.eps, (const S*)a.residual, (S*)a.residual_out);
}
template <typename T, int RPW, bool RES>
static void launch_fwd_rows(hipStream_t s, const FwdArgs& a, int np) {
    if (np == 8) launch_fwd_rows_np<T, RPW, RES, 8>(s, a);
    else if (np == 4) launch_fwd_rows_np<T, RPW, RES, 4>(s, a);
    else launch_fwd_rows_np<T, RPW, RES, 0>(s, a);
}

// waves (or wider teams) that walk rows with the next row in flight: as many workgroups as are resident at once
template <typename T, int TPR, bool RES, int NP>
static void launch_fwd_walk_np(hipStream_t s, const FwdArgs& a) {
    typedef typename T::storage_t S;
    constexpr int block = TPR > 256 ? TPR : 256;
    const void* kernel = (const void*)ck::rmsnorm_fwd_kernel<T, TPR, RES, NP>;
    int64_t grid = (int64_t)cu_count() * resident_blocks(kernel, block);
    const int64_t need = ck_ceil_div(a.B, block / TPR);
    if (grid > need) grid = need;
    hipLaunchKernelGGL((ck::rmsnorm_fwd_kernel<T, TPR, RES, NP>), dim3((unsigned)grid), dim3(block), 0, s, (const S*)a.x,
                       (const S*)a.weight, (S*)a.output, a.rstd, a.B, a.H, a.eps, (const S*)a.residual, (S*)a.residual_out);
}
template <typename T, int TPR, bool RES>
static void launch_fwd_walk(hipStream_t s, const FwdArgs& a, int np) {
    if (np == 8) launch_fwd_walk_np<T, TPR, RES, 8>(s, a);
    else if (np == 4) launch_fwd_walk_np<T, TPR, RES, 4>(s, a);
    else if (np == 2) launch_fwd_walk_np<T, TPR, RES, 2>(s, a);
    else launch_fwd_walk_np<T, TPR, RES, 0>(s, a);
}

// the fast paths of both forward entry points (tpr = 64, 256; 1024 without a residual)
template <typename T, bool RES>
static void launch_fwd_fast(hipStream_t s, const FwdArgs& a, int tpr, int dtype, int block_size_b) {
    const int np = exact_packs(a.H, dtype, tpr);
    const int rows = block_size_b == 0 ? fwd_default_rows(a.H, dtype) : block_size_b;
    if (tpr == 64 && rows == 1) launch_fwd_rows<T, 1, RES>(s, a, np);
    else if (tpr == 64 && rows < 8) launch_fwd_rows<T, 2, RES>(s, a, np);
    else if (tpr == 64) launch_fwd_walk<T, 64, RES>(s, a, np);
    else if (tpr == 256) launch_fwd_walk<T, 256, RES>(s, a, np);
    else launch_fwd_walk_np<T, 1024, false, 0>(s, a);
}

extern "C" int ck_rmsnorm_forward(const void* x, const void* weight, void* output, float* rstd, int64_t B, int64_t H,
                                  float eps, int dtype, int block_size_b, void* stream) {
    if (block_size_b < 0) return CK_ERR_SHAPE;
    if (B < 0 || H < 0 || H > 65536) return CK_ERR_SHAPE;
    if (B == 0 || H == 0) return CK_OK;
    if (!x || !output) return CK_ERR_NULL;
    if (!ck_aligned_elem(x, dtype) || !ck_aligned_elem(output, dtype) || (weight && !ck_aligned_elem(weight, dtype)))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = ck_aligned16(x) && ck_aligned16(output) && (!weight || ck_aligned16(weight));
    const int tpr = aligned ? fast_tpr(H, dtype) : 0;
    const FwdArgs a = {x, nullptr, weight, output, nullptr, rstd, B, (int)H, eps};
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        if (tpr != 0) {
            launch_fwd_fast<T, false>(s, a, tpr, dtype, block_size_b);
        } else {
            const int64_t grid = B < 65536 ? B : 65536;
            hipLaunchKernelGGL((ck::rmsnorm_fwd_generic_kernel<T>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)x,
                               (const S*)weight, (S*)output, rstd, B, (int)H, eps);
        }
    });
    return ck_launch_status();
}

extern "C" int ck_residual_rmsnorm_forward(const void* x, const void* residual, const void* weight, void* output,
                                           void* residual_out, float* rstd, int64_t B, int64_t H, float eps, int dtype,
                                           int block_size_b, void* stream) {
    if (block_size_b < 0) return CK_ERR_SHAPE;
    if (B < 0 || H < 0 || H > 65536) return CK_ERR_SHAPE;
    if (B == 0 || H == 0) return CK_OK;
    if (!x || !residual || !output || !residual_out) return CK_ERR_NULL;
    if (!ck_aligned_elem(x, dtype) || !ck_aligned_elem(residual, dtype) || !ck_aligned_elem(output, dtype) ||
        !ck_aligned_elem(residual_out, dtype) || (weight && !ck_aligned_elem(weight, dtype)))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = ck_aligned16(x) && ck_aligned16(residual) && ck_aligned16(output) && ck_aligned16(residual_out) &&
                         (!weight || ck_aligned16(weight));
    const int tpr = aligned ? fast_tpr(H, dtype) : 0;
    if (tpr != 64 && tpr != 256) {
        // rows outside the register budget of the one-pass kernel (or unaligned): the sum, then the normalisation
        const int st = ck_add_tensor_forward(x, residual, residual_out, B * H, dtype, 256, stream);
        if (st != CK_OK) return st;
        return ck_rmsnorm_forward(residual_out, weight, output, rstd, B, H, eps, dtype, block_size_b, stream);
    }
    const FwdArgs a = {x, residual, weight, output, residual_out, rstd, B, (int)H, eps};
    CK_DISPATCH_DTYPE(dtype, { launch_fwd_fast<T, true>(s, a, tpr, dtype, block_size_b); });
    return ck_launch_status();
}

// Workspace layout.  Fast path: room for teams x H fp32 partial rows (one per workgroup is used, then kReduceSplits).  Generic path: B fp32 rstd values, then
// kColSegments x H_padded fp32 partial rows.  The query returns the larger of the two.
static int64_t padded_h(int64_t H) { return (H + 3) / 4 * 4; }

extern "C" int64_t ck_rmsnorm_backward_workspace_size(int64_t B, int64_t H) {
    if (B <= 0 || H <= 0) return 0;
    int64_t teams = 1;
    for (int tpr : {64, 256, 1024}) {
        const int64_t t = bwd_teams(B, tpr, tpr == 64 ? 2 : 1);
        if (t > teams) teams = t;
    }
    const int64_t fast = (teams + kReduceSplits) * H * 4;
    const int64_t generic = (B + 3) / 4 * 16 + (int64_t)ck::kColSegments * padded_h(H) * 4;
    return fast > generic ? fast : generic;
}

struct BwdArgs {
    const void *x, *weight, *dy;
    const float* rstd;
    void* dx;
    float* ws;
    int64_t B;
    int H;
    float eps;
};

template <typename T, int TPR, int NP, bool W, bool SS>
static void launch_bwd_one(unsigned grid, int block, hipStream_t s, const BwdArgs& a) {
    typedef typename T::storage_t S;
    hipLaunchKernelGGL((ck::rmsnorm_bwd_kernel<T, TPR, W, NP, SS>), dim3(grid), dim3(block), 0, s, (const S*)a.x,
                       (const S*)a.weight, (const S*)a.dy, a.rstd, (S*)a.dx, a.ws, a.B, a.H, a.eps);
}
template <typename T, int TPR, int NP>
static void launch_bwd_np(unsigned grid, int block, hipStream_t s, const BwdArgs& a) {
    if constexpr (TPR == 1024) {
        // (the form that never sums the squares spills at 128 registers per lane and is not compiled)
        if (a.weight) launch_bwd_one<T, TPR, NP, true, true>(grid, block, s, a);
        else launch_bwd_one<T, TPR, NP, false, true>(grid, block, s, a);
    } else {
        const bool ss = a.rstd == nullptr;  // 1 / rms was not saved: the kernel forms it
        if (a.weight) {
            if (ss) launch_bwd_one<T, TPR, NP, true, true>(grid, block, s, a);
            else launch_bwd_one<T, TPR, NP, true, false>(grid, block, s, a);
        } else {
            if (ss) launch_bwd_one<T, TPR, NP, false, true>(grid, block, s, a);
            else launch_bwd_one<T, TPR, NP, false, false>(grid, block, s, a);
        }
    }
}
template <typename T, int TPR>
static void launch_bwd(unsigned grid, int block, hipStream_t s, const BwdArgs& a, int np) {
    if (np == 8) launch_bwd_np<T, TPR, 8>(grid, block, s, a);
    else if (np == 4) launch_bwd_np<T, TPR, 4>(grid, block, s, a);
    else launch_bwd_np<T, TPR, 0>(grid, block, s, a);
}
template <typename T, int NP, bool W, bool SS>
static void launch_bwd_two_one(unsigned grid, hipStream_t s, const BwdArgs& a) {
    typedef typename T::storage_t S;
    hipLaunchKernelGGL((ck::rmsnorm_bwd_two_kernel<T, W, NP, SS>), dim3(grid), dim3(256), 0, s, (const S*)a.x,
                       (const S*)a.weight, (const S*)a.dy, a.rstd, (S*)a.dx, a.ws, a.B, a.H, a.eps);
}
template <typename T, int NP>
static void launch_bwd_two_np(unsigned grid, hipStream_t s, const BwdArgs& a) {
    typedef typename T::storage_t S;
    const bool ss = a.rstd == nullptr;
    if (a.weight) {
        // (16-bit rows of a generic packet count with a weight never come here - see two_fits - and are not compiled)
        if constexpr (NP != 0 || sizeof(S) == 4) {
            if (ss) launch_bwd_two_one<T, NP, true, true>(grid, s, a);
            else launch_bwd_two_one<T, NP, true, false>(grid, s, a);
        }
    } else {
        if (ss) launch_bwd_two_one<T, NP, false, true>(grid, s, a);
        else launch_bwd_two_one<T, NP, false, false>(grid, s, a);
    }
}

extern "C" int ck_rmsnorm_backward(const void* x, const void* weight, const void* output_grad, const float* rstd,
                                   void* x_grad, void* weight_grad, void* workspace, int64_t workspace_bytes, int64_t B,
                                   int64_t H, float eps, int dtype, int block_size_b, void* stream) {
    if (B < 0 || H < 0 || H > 65536 || block_size_b < 0) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    hipStream_t s = (hipStream_t)stream;
    if (B == 0 || H == 0) {
        // an empty batch still defines dweight = 0
        if (weight && weight_grad && H > 0) {
            // (a launch, not a memset: the call may be recorded into a graph)
            CK_DISPATCH_DTYPE(dtype, {
                typedef typename T::storage_t S;
                hipLaunchKernelGGL((ck::rmsnorm_dw_reduce_generic_kernel<T>), dim3((unsigned)ck_ceil_div(H, 256)), dim3(256), 0,
                                   s, (const float*)nullptr, (S*)weight_grad, 0, (int)H, (int)H);
            });
            return ck_launch_status();
        }
        return CK_OK;
    }
    if (!x || !output_grad || !x_grad) return CK_ERR_NULL;
    if (weight && !weight_grad) return CK_ERR_NULL;
    const void* ptrs[5] = {x, output_grad, x_grad, weight, weight_grad};
    bool aligned = true;
    for (const void* p : ptrs) {
        if (!p) continue;
        if (!ck_aligned_elem(p, dtype)) return CK_ERR_ALIGN;
        aligned = aligned && ck_aligned16(p);
    }
    if (weight) {
        if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return CK_ERR_WORKSPACE;
        if (workspace_bytes < ck_rmsnorm_backward_workspace_size(B, H)) return CK_ERR_WORKSPACE;
    }
    const int tpr = aligned ? fast_tpr(H, dtype) : 0;
    float* ws = (float*)workspace;

    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        if (tpr != 0) {
            const int np = tpr == 1024 ? 0 : exact_packs(H, dtype, tpr);
            const int64_t row_packs = H / (dtype == CK_F32 ? 4 : 8);
            // 16-bit rows with a weight that are neither 1, 2 nor 4 packets per lane: the two-workgroup form would
            // spill (it is compiled for 256 registers), the one-workgroup form holds them
            const bool two_fits = !(weight && dtype != CK_F32 && (np == 0 || np == 8) && row_packs != 64);
            const bool two = tpr == 64 && two_fits &&
                             (block_size_b == 0 ? bwd_default_variant(H, dtype) : block_size_b) == 1;
            const int teams = bwd_teams(B, tpr, two ? 2 : 1);
            const int block = tpr > 256 ? tpr : 256;
            const unsigned grid = (unsigned)(teams / (block / tpr));
            const BwdArgs a = {x, weight, output_grad, rstd, x_grad, ws, B, (int)H, eps};
            if (two) {
                // (the branch-free form for eight packets per lane needs more than the 256 registers two waves per
                // SIMD leave; the short exact rows are the ones this variant is the default for)
                if (np == 4) launch_bwd_two_np<T, 4>(grid, s, a);
                else if (np == 2) launch_bwd_two_np<T, 2>(grid, s, a);
                else if (row_packs == 64) launch_bwd_two_np<T, 1>(grid, s, a);
                else launch_bwd_two_np<T, 0>(grid, s, a);
            } else if (tpr == 64) launch_bwd<T, 64>(grid, block, s, a, np);
            else if (tpr == 256) launch_bwd<T, 256>(grid, block, s, a, np);
            else launch_bwd_np<T, 1024, 0>(grid, block, s, a);
            if (weight) {
                // one partial row per workgroup -> (kReduceSplits rows, fp32, behind the partial rows ->) dweight
                const int rows = (int)grid;
                const int splits = rows >= 32 * kReduceSplits ? kReduceSplits : 1;
                float* second = ws + (int64_t)teams * H;
                if (splits > 1) {
                    hipLaunchKernelGGL((ck::rmsnorm_dw_reduce_kernel<T>), dim3((unsigned)ck_ceil_div(H, 16), splits),
                                       dim3(64), 0, s, ws, (S*)nullptr, second, rows, (int)H);
                    hipLaunchKernelGGL((ck::rmsnorm_dw_reduce_kernel<T>), dim3((unsigned)ck_ceil_div(H, 16), 1), dim3(64),
                                       0, s, second, (S*)weight_grad, (float*)nullptr, splits, (int)H);
                } else {
                    hipLaunchKernelGGL((ck::rmsnorm_dw_reduce_kernel<T>), dim3((unsigned)ck_ceil_div(H, 16), 1), dim3(64),
                                       0, s, ws, (S*)weight_grad, (float*)nullptr, rows, (int)H);
                }
            }
        } else {
            const int64_t grid = B < 65536 ? B : 65536;
            float* rstd_ws = weight ? ws : nullptr;
            hipLaunchKernelGGL((ck::rmsnorm_bwd_generic_kernel<T>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)x,
                               (const S*)weight, (const S*)output_grad, rstd, (S*)x_grad, rstd_ws, B, (int)H, eps);
            if (weight) {
                const int hp = (int)padded_h(H);
                float* partial = ws + (B + 3) / 4 * 4;
                hipLaunchKernelGGL((ck::rmsnorm_dw_columns_kernel<T>),
                                   dim3((unsigned)ck_ceil_div(hp, 256), ck::kColSegments), dim3(256), 0, s, (const S*)x,
                                   (const S*)output_grad, rstd_ws, partial, B, (int)H, hp);
                hipLaunchKernelGGL((ck::rmsnorm_dw_reduce_generic_kernel<T>), dim3((unsigned)ck_ceil_div(H, 256)),
                                   dim3(256), 0, s, partial, (S*)weight_grad, ck::kColSegments, (int)H, hp);
            }
        }
    });
    return ck_launch_status();
}
