// Stable LSD radix sort of (key, value) pairs spread over the whole GPU: three kernels per pass.
//   histogram : every wave owns kGridSortWaveKeys consecutive pairs, groups them by digit with ballots
//               (wave_match) and writes its per-digit counts to hist[digit][wave]
//   scan      : one workgroup turns hist into exclusive offsets in (digit, wave) order
//   scatter   : every wave ranks its pairs again and stores them at offset + rank
// The single-workgroup sort in ck_block_sort.h is faster for a handful of bins (expert ids); with hundreds of
// bins its scattered stores all leave from one compute unit, which is what this version avoids.
#pragma once

#include "ck_device.h"

namespace ck {

constexpr int kGridSortBatches = 8;  // batches of 64 pairs per wave
constexpr int kGridSortWaveKeys = kGridSortBatches * CK_WAVE;
constexpr int kGridSortMaxBits = 9;

__host__ __device__ static inline int grid_sort_waves(int64_t n) {
    return (int)((n + kGridSortWaveKeys - 1) / kGridSortWaveKeys);
}

constexpr int kGridSortBlockWaves = 4;  // workgroup = 256 lanes
struct GridSortShared {
    uint32_t bins[kGridSortBlockWaves][1 << kGridSortMaxBits];  // one row per wave: no sharing, no atomics
};

// Load : (int i, uint32_t& key, uint32_t& val)
template <typename Load>
__device__ __forceinline__ void grid_sort_histogram(GridSortShared& sh, int n, int shift, int bits,
                                                    uint32_t* __restrict__ hist, int num_waves, Load load) {
    const int lane = lane_id();
    const int wave = threadIdx.x / CK_WAVE;
    const int gw = blockIdx.x * kGridSortBlockWaves + wave;
    if (gw >= num_waves) return;
    const uint32_t mask = (1u << bits) - 1u;
    const int nbins = 1 << bits;
    const int begin = gw * kGridSortWaveKeys;
    uint32_t keys[kGridSortBatches], vals[kGridSortBatches];
#pragma unroll
    for (int u = 0; u < kGridSortBatches; ++u) {
        const int i = begin + u * CK_WAVE + lane;
        keys[u] = 0;
        vals[u] = 0;
        if (i < n) load(i, keys[u], vals[u]);
    }
    uint32_t* bins = sh.bins[wave];
    for (int d = lane; d < nbins; d += CK_WAVE) bins[d] = 0;
#pragma unroll
    for (int u = 0; u < kGridSortBatches; ++u) {
        const int i = begin + u * CK_WAVE + lane;
        const bool valid = i < n;
        const uint32_t digit = (keys[u] >> shift) & mask;
        const uint64_t m = wave_match(digit, bits, valid);
        // groups of one batch hold different digits, batches follow each other in program order
        if (valid && (m & lanemask_lt()) == 0) bins[digit] += (uint32_t)__popcll(m);
    }
    CK_WAVE_LOCKSTEP();
    for (int d = lane; d < nbins; d += CK_WAVE) hist[(int64_t)d * num_waves + gw] = bins[d];
}

// in place: hist[k] <- sum of hist[0 .. k-1], k over nbins * num_waves entries; one workgroup of 1024 lanes.
// Each wave owns a contiguous slice and walks it 64 entries at a time (coalesced).  A slice of up to
// 64 * kScanHeld entries is read once, all batches requested together, and scanned out of registers; longer
// slices take two sweeps of kScanAhead batches (totals first, exclusive sums second).
constexpr int kScanAhead = 8;
constexpr int kScanHeld = 32;
__device__ __forceinline__ void grid_sort_scan(uint32_t* __restrict__ hist, int total) {
    __shared__ uint32_t wave_total[16];
    const int lane = lane_id();
    const int wave = threadIdx.x / CK_WAVE;
    const int per_wave = ((total + 15) / 16 + CK_WAVE - 1) / CK_WAVE * CK_WAVE;
    const int begin = min(wave * per_wave, total);
    const int end = min(begin + per_wave, total);
    if (per_wave <= CK_WAVE * kScanHeld) {
        uint32_t v[kScanHeld];
        uint32_t sum = 0;
#pragma unroll
        for (int u = 0; u < kScanHeld; ++u) {
            const int i = begin + u * CK_WAVE + lane;
            v[u] = i < end ? hist[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < kScanHeld; ++u) sum += v[u];
        sum = (uint32_t)wave_sum_i((int)sum);
        if (lane == 0) wave_total[wave] = sum;
        __syncthreads();
        uint32_t carry = 0;
        for (int w = 0; w < wave; ++w) carry += wave_total[w];
#pragma unroll
        for (int u = 0; u < kScanHeld; ++u) {
            const int i = begin + u * CK_WAVE + lane;
            if (begin + u * CK_WAVE >= end) break;  // wave-uniform
            const uint32_t incl = (uint32_t)wave_inclusive_scan_i((int)v[u]);
            if (i < end) hist[i] = carry + incl - v[u];
            carry += __shfl(incl, CK_WAVE - 1, CK_WAVE);
        }
        return;
    }
    uint32_t sum = 0;
    for (int g0 = begin; g0 < end; g0 += CK_WAVE * kScanAhead) {
#pragma unroll
        for (int u = 0; u < kScanAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            if (i < end) sum += hist[i];
        }
    }
    sum = (uint32_t)wave_sum_i((int)sum);
    if (lane == 0) wave_total[wave] = sum;
    __syncthreads();
    uint32_t carry = 0;
    for (int w = 0; w < wave; ++w) carry += wave_total[w];
    for (int g0 = begin; g0 < end; g0 += CK_WAVE * kScanAhead) {
        uint32_t v[kScanAhead];
#pragma unroll
        for (int u = 0; u < kScanAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            v[u] = i < end ? hist[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < kScanAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            const uint32_t incl = (uint32_t)wave_inclusive_scan_i((int)v[u]);
            if (i < end) hist[i] = carry + incl - v[u];
            carry += __shfl(incl, CK_WAVE - 1, CK_WAVE);
        }
    }
}

// Store : (int pos, uint32_t key, uint32_t val)
template <typename Load, typename Store>
__device__ __forceinline__ void grid_sort_scatter(GridSortShared& sh, int n, int shift, int bits,
                                                  const uint32_t* __restrict__ offsets, int num_waves, Load load,
                                                  Store store) {
    const int lane = lane_id();
    const int wave = threadIdx.x / CK_WAVE;
    const int gw = blockIdx.x * kGridSortBlockWaves + wave;
    if (gw >= num_waves) return;
    const uint32_t mask = (1u << bits) - 1u;
    const int nbins = 1 << bits;
    const int begin = gw * kGridSortWaveKeys;
    uint32_t keys[kGridSortBatches], vals[kGridSortBatches];
#pragma unroll
    for (int u = 0; u < kGridSortBatches; ++u) {
        const int i = begin + u * CK_WAVE + lane;
        keys[u] = 0;
        vals[u] = 0;
        if (i < n) load(i, keys[u], vals[u]);
    }
    uint32_t* next = sh.bins[wave];  // running offset of each bin for this wave
    for (int d = lane; d < nbins; d += CK_WAVE) next[d] = offsets[(int64_t)d * num_waves + gw];
#pragma unroll
    for (int u = 0; u < kGridSortBatches; ++u) {
        const int i = begin + u * CK_WAVE + lane;
        const bool valid = i < n;
        const uint32_t digit = (keys[u] >> shift) & mask;
        const uint64_t m = wave_match(digit, bits, valid);
        const uint64_t lower = m & lanemask_lt();
        uint32_t pos = 0;
        if (valid) pos = next[digit] + (uint32_t)__popcll(lower);
        // every lane of the group has read the offset before its first lane advances it
        CK_WAVE_LOCKSTEP();
        if (valid && lower == 0) next[digit] += (uint32_t)__popcll(m);
        if (valid) store((int)pos, keys[u], vals[u]);
    }
}

}  // namespace ck
