// Stable least-significant-digit radix sort of (key, value) pairs executed by ONE workgroup of
// kSortThreads lanes (16 wavefronts), built on wave64 ballots:
//   - each wavefront owns a contiguous slice of the input and walks it 64 keys at a time, in order;
//   - lanes holding the same digit find each other with one ballot per digit bit (wave_match);
//     popcounts of that mask give the group size (histogram) and the lane's rank inside the group;
//   - per-wave digit histograms live in LDS, so no atomics are needed and the result is stable.
// Used for the MoE expert sort (1 pass for up to 256 experts) and for sorting token ids in the
// embedding backward (3 passes for a 17-bit vocabulary).  The sizes it is used at (1e4..1e6 keys) keep
// a one-workgroup sort within tens of microseconds and save the launches a multi-kernel sort needs.
#pragma once

#include "ck_device.h"

namespace ck {

constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / CK_WAVE;
constexpr int kSortMaxBits = 8;
constexpr int kSortBins = 1 << kSortMaxBits;
constexpr int kSortAhead = 16;  // batches of 64 keys requested together

struct SortShared {
    int hist[kSortWaves][kSortBins];  // per-wave digit counts, then per-wave exclusive offsets
    int digit_base[kSortBins];        // exclusive prefix of the digit totals
};

// number of significant bits of keys in [0, num_keys)
__host__ __device__ static inline int ck_key_bits(int64_t num_keys) {
    int bits = 1;
    while (bits < 32 && ((int64_t)1 << bits) < num_keys) ++bits;
    return bits;
}
__host__ __device__ static inline int ck_sort_passes(int key_bits) { return (key_bits + kSortMaxBits - 1) / kSortMaxBits; }

// One pass over `n` pairs on the digit (key >> shift) & ((1 << bits) - 1).
//   Load  : (int i, uint32_t& key, uint32_t& val)   reads pair i of this pass's input
//   Store : (int pos, uint32_t key, uint32_t val)   writes the pair to its sorted position
// Every lane of the workgroup must call it; it starts and ends with a barrier, so global writes of the
// previous pass are visible to this one and this pass's writes are visible afterwards.
template <typename Load, typename Store>
__device__ __forceinline__ void block_radix_pass(SortShared& sh, int n, int shift, int bits, Load load, Store store) {
    const int wave = threadIdx.x / CK_WAVE;
    const int lane = lane_id();
    const uint32_t mask = (1u << bits) - 1u;
    const int nbins = 1 << bits;
    // slice of this wave: a multiple of 64 keys so that batches never straddle two waves
    const int per_wave = ((n + kSortWaves - 1) / kSortWaves + CK_WAVE - 1) / CK_WAVE * CK_WAVE;
    const int begin = min(wave * per_wave, n);
    const int end = min(begin + per_wave, n);

    __syncthreads();
    for (int d = lane; d < nbins; d += CK_WAVE) sh.hist[wave][d] = 0;
    // (each wave touches only its own histogram row: program order inside the wave is enough)

    // keys are fetched kSortAhead batches at a time so that their memory latency is paid once per group, not
    // once per batch; the batches of a group are then ranked one after the other, in order
    for (int g0 = begin; g0 < end; g0 += CK_WAVE * kSortAhead) {
        uint32_t keys[kSortAhead], vals[kSortAhead];
#pragma unroll
        for (int u = 0; u < kSortAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            keys[u] = 0;
            vals[u] = 0;
            if (i < end) load(i, keys[u], vals[u]);
        }
#pragma unroll
        for (int u = 0; u < kSortAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            const bool valid = i < end;
            const uint32_t digit = (keys[u] >> shift) & mask;
            const uint64_t m = wave_match(digit, bits, valid);
            if (valid && (m & lanemask_lt()) == 0) sh.hist[wave][digit] += __popcll(m);
        }
    }
    __syncthreads();

    // exclusive prefix over the waves for each digit, digit totals, then exclusive prefix over digits
    for (int d = threadIdx.x; d < nbins; d += kSortThreads) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const int c = sh.hist[w][d];
            sh.hist[w][d] = run;
            run += c;
        }
        sh.digit_base[d] = run;
    }
    __syncthreads();
    if (wave == 0) {
        // 256 bins = 4 per lane: local prefix + wave scan of the lane sums
        int t[kSortBins / CK_WAVE];
        int local = 0;
#pragma unroll
        for (int j = 0; j < kSortBins / CK_WAVE; ++j) {
            const int d = lane * (kSortBins / CK_WAVE) + j;
            t[j] = d < nbins ? sh.digit_base[d] : 0;
            local += t[j];
        }
        int excl = wave_inclusive_scan_i(local) - local;
#pragma unroll
        for (int j = 0; j < kSortBins / CK_WAVE; ++j) {
            const int d = lane * (kSortBins / CK_WAVE) + j;
            if (d < nbins) sh.digit_base[d] = excl;
            excl += t[j];
        }
    }
    __syncthreads();

    for (int g0 = begin; g0 < end; g0 += CK_WAVE * kSortAhead) {
        uint32_t keys[kSortAhead], vals[kSortAhead];
#pragma unroll
        for (int u = 0; u < kSortAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            keys[u] = 0;
            vals[u] = 0;
            if (i < end) load(i, keys[u], vals[u]);
        }
#pragma unroll
        for (int u = 0; u < kSortAhead; ++u) {
            const int i = g0 + u * CK_WAVE + lane;
            const bool valid = i < end;
            const uint32_t digit = (keys[u] >> shift) & mask;
            const uint64_t m = wave_match(digit, bits, valid);
            const uint64_t lower = m & lanemask_lt();
            int pos = 0;
            if (valid) pos = sh.digit_base[digit] + sh.hist[wave][digit] + __popcll(lower);
            // all lanes have read the running offset before the group's first lane advances it
            CK_WAVE_LOCKSTEP();
            if (valid && lower == 0) sh.hist[wave][digit] += __popcll(m);
            if (valid) store(pos, keys[u], vals[u]);
        }
    }
    __threadfence_block();
    __syncthreads();
}

}  // namespace ck
