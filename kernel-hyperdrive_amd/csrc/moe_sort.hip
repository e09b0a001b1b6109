// Integer front end of the MoE layer on gfx950: histogram of expert ids, stable expert sort with
// positions, and inclusive expert offsets.  All results are integers and bit-exact by construction:
//   - ck_contiguous_count : bincount with a fixed number of bins
//       (cute_kernels/kernels/contiguous_count/triton_implementation/kernels_forward.py:13-66)
//   - ck_moe_sort         : selected_experts.flatten().sort() + bincount + cumsum
//       (cute_kernels/kernels/scattermoe/triton_implementation/__init__.py:80-81), with ties kept in
//       input order (stable), which torch's default sort does not promise
//   - ck_offsets_from_sorted : cumsum(bincount) recovered from already-sorted ids.
#include <mutex>

#include "ck_block_sort.h"
#include "ck_grid_sort.h"

namespace ck {

template <bool I32>
__device__ __forceinline__ int64_t load_id(const void* p, int64_t i) {
    return I32 ? (int64_t) reinterpret_cast<const int32_t*>(p)[i] : reinterpret_cast<const int64_t*>(p)[i];
}

// ---- histogram -------------------------------------------------------------------------------
constexpr int kCountLdsBins = 4096;

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Each wave walks its slice 64 ids at a time; lanes with equal ids are grouped by ballots and the first
// lane of a group adds the group size to the workgroup's LDS bins (integer LDS atomics: exact in any
// order).  Bins are flushed to global with integer atomics.  bins <= kCountLdsBins.
template <bool I32>
__global__ void __launch_bounds__(256)
    count_kernel(const void* __restrict__ x, int32_t* __restrict__ out, int64_t n, int bins, int key_bits) {
    __shared__ int lds[kCountLdsBins];
    for (int c = threadIdx.x; c < bins; c += blockDim.x) lds[c] = 0;
    __syncthreads();
    const int64_t per_block = (n + gridDim.x - 1) / gridDim.x;
    const int64_t b0 = (int64_t)blockIdx.x * per_block;
    const int64_t b1 = b0 + per_block < n ? b0 + per_block : n;
    // whole batches of blockDim ids; the trip count is uniform over the workgroup
    for (int64_t i0 = b0; i0 < b1; i0 += blockDim.x) {
        const int64_t i = i0 + threadIdx.x;
        int64_t v = -1;
        if (i < b1) v = load_id<I32>(x, i);
        const bool valid = v >= 0 && v < bins;
        const uint64_t m = wave_match((uint32_t)v, key_bits, valid);
        if (valid && (m & lanemask_lt()) == 0) atomicAdd(&lds[(int)v], __popcll(m));
    }
    __syncthreads();
    for (int c = threadIdx.x; c < bins; c += blockDim.x) {
        const int v = lds[c];
        if (v != 0) atomicAdd(&out[c], v);
    }
}

// bins > kCountLdsBins: integer atomics straight to global
template <bool I32>
__global__ void __launch_bounds__(256)
    count_global_kernel(const void* __restrict__ x, int32_t* __restrict__ out, int64_t n, int64_t bins) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t v = load_id<I32>(x, i);
    if (v >= 0 && v < bins) atomicAdd(&out[v], 1);
}

// ---- expert sort -----------------------------------------------------------------------------
// workspace: 4 arrays of M uint32 (two key/value ping-pong pairs), used only when more than one pass
// is needed (E > 256).
template <bool I32>
__global__ void __launch_bounds__(kSortThreads)
    moe_sort_kernel(const void* __restrict__ ids, int64_t* __restrict__ sorted_ids, int64_t* __restrict__ sorted_pos,
                    int64_t* __restrict__ offsets, uint32_t* __restrict__ ws, int M, int E, int key_bits) {
    __shared__ SortShared sh;
    const int passes = ck_sort_passes(key_bits);
    const int bits_per_pass = (key_bits + passes - 1) / passes;
    uint32_t* kbuf[2] = {ws, ws + 2 * (int64_t)M};
    uint32_t* vbuf[2] = {ws + (int64_t)M, ws + 3 * (int64_t)M};

    for (int p = 0; p < passes; ++p) {
        const int shift = p * bits_per_pass;
        const int bits = min(bits_per_pass, key_bits - shift);
        const bool first = p == 0, last = p == passes - 1;
        const uint32_t* kin = kbuf[(p + 1) & 1];
        const uint32_t* vin = vbuf[(p + 1) & 1];
        uint32_t* kout = kbuf[p & 1];
        uint32_t* vout = vbuf[p & 1];
        auto load = [&](int i, uint32_t& k, uint32_t& v) {
            if (first) {
                k = (uint32_t)load_id<I32>(ids, i);
                v = (uint32_t)i;
            } else {
                k = kin[i];
                v = vin[i];
            }
        };
        auto store = [&](int pos, uint32_t k, uint32_t v) {
            if (last) {
                sorted_ids[pos] = (int64_t)k;
                sorted_pos[pos] = (int64_t)v;
            } else {
                kout[pos] = k;
                vout[pos] = v;
            }
        };
        block_radix_pass(sh, M, shift, bits, load, store);
    }

    // inclusive offsets from the boundaries of the sorted ids: offsets[e] = #{ids <= e}
    if (M == 0) {
        for (int e = threadIdx.x; e < E; e += kSortThreads) offsets[e] = 0;
        return;
    }
    for (int i = threadIdx.x; i < M; i += kSortThreads) {
        const int64_t k = sorted_ids[i];
        const int64_t next = (i + 1 < M) ? sorted_ids[i + 1] : (int64_t)E;
        if (i == 0)
            for (int64_t e = 0; e < k && e < E; ++e) offsets[e] = 0;
        for (int64_t e = k; e < next && e < E; ++e) offsets[e] = (int64_t)i + 1;
    }
}

// ---- the same sort spread over the GPU -----------------------------------------------------------
// One workgroup sorts 16K ids in ~37 us (the three launches below: 15) and needs ~200 us for 100K: from
// kGridSortFrom ids on (and up to 2^kGridSortMaxBits experts, one radix pass) the three kernels of
// ck_grid_sort.h take over.  Ids become the
// keys, positions the values; the scatter kernel also derives the expert offsets from the scanned histogram
// (the exclusive offset of bin e + 1 for the first wave = number of ids <= e).
constexpr int64_t kGridSortFrom = 16384;

template <bool I32>
struct ExpertIdLoader {
    const void* ids;
    __device__ __forceinline__ void operator()(int i, uint32_t& key, uint32_t& val) const {
        key = (uint32_t)load_id<I32>(ids, i);
        val = (uint32_t)i;
    }
};
struct SortedStorer {
    int64_t* sorted_ids;
    int64_t* sorted_pos;
    __device__ __forceinline__ void operator()(int pos, uint32_t key, uint32_t val) const {
        sorted_ids[pos] = (int64_t)key;
        sorted_pos[pos] = (int64_t)val;
    }
};

template <bool I32>
__global__ void __launch_bounds__(256)
    moe_grid_hist_kernel(ExpertIdLoader<I32> load, int M, int bits, uint32_t* __restrict__ hist, int num_waves) {
    __shared__ GridSortShared sh;
    grid_sort_histogram(sh, M, 0, bits, hist, num_waves, load);
}

__global__ void __launch_bounds__(1024) moe_grid_scan_kernel(uint32_t* __restrict__ hist, int total) {
    grid_sort_scan(hist, total);
}

template <bool I32>
__global__ void __launch_bounds__(256)
    moe_grid_scatter_kernel(ExpertIdLoader<I32> load, SortedStorer store, int M, int bits,
                            const uint32_t* __restrict__ scanned, int num_waves, int64_t* __restrict__ offsets, int E) {
    __shared__ GridSortShared sh;
    if (blockIdx.x == 0) {
        const int nbins = 1 << bits;
        for (int e = threadIdx.x; e < E; e += blockDim.x)
            offsets[e] = e + 1 < nbins ? (int64_t)scanned[(int64_t)(e + 1) * num_waves] : (int64_t)M;
    }
    grid_sort_scatter(sh, M, 0, bits, scanned, num_waves, load, store);
}

__global__ void __launch_bounds__(256)
    offsets_from_sorted_kernel(const int64_t* __restrict__ sorted_ids, int64_t* __restrict__ offsets, int64_t M,
                               int64_t E) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (M == 0) {
        for (int64_t e = t; e < E; e += stride) offsets[e] = 0;
        return;
    }
    for (int64_t i = t; i < M; i += stride) {
        const int64_t k = sorted_ids[i];
        const int64_t next = (i + 1 < M) ? sorted_ids[i + 1] : E;
        if (i == 0)
            for (int64_t e = 0; e < k && e < E; ++e) offsets[e] = 0;
        for (int64_t e = k; e < next && e < E; ++e) offsets[e] = i + 1;
    }
}

}  // namespace ck

extern "C" int ck_contiguous_count(const void* x, int x_is_i32, int32_t* output, int64_t n, int64_t size,
                                   void* stream) {
    if (n < 0 || size < 0 || size > 0x7fffffff) return CK_ERR_SHAPE;
    if (size == 0) return CK_OK;
    if (!output || (n > 0 && !x)) return CK_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(ck::fill_i32_kernel, dim3((unsigned)ck_ceil_div(size, 256)), dim3(256), 0, s, output, size, 0);
    if (n > 0) {
        if (size <= ck::kCountLdsBins) {
            int64_t blocks = ck_ceil_div(n, 256 * 16);
            if (blocks > 1024) blocks = 1024;
            const int key_bits = ck::ck_key_bits(size);
            if (x_is_i32)
                hipLaunchKernelGGL(ck::count_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, x, output, n,
                                   (int)size, key_bits);
            else
                hipLaunchKernelGGL(ck::count_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, x, output, n,
                                   (int)size, key_bits);
        } else {
            const int64_t blocks = ck_ceil_div(n, 256);
            if (blocks > 0x7fffffff) return CK_ERR_SHAPE;
            if (x_is_i32)
                hipLaunchKernelGGL(ck::count_global_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, x, output, n,
                                   size);
            else
                hipLaunchKernelGGL(ck::count_global_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, x, output,
                                   n, size);
        }
    }
    return ck_launch_status();
}

static bool use_grid_sort(int64_t M, int64_t E) {
    return M >= ck::kGridSortFrom && ck::ck_key_bits(E) <= ck::kGridSortMaxBits;
}

extern "C" int64_t ck_moe_sort_workspace_size(int64_t M, int64_t E) {
    if (M <= 0 || E <= 0) return 0;
    if (use_grid_sort(M, E))  // histogram [bins][waves]
        return ((int64_t)1 << ck::ck_key_bits(E)) * ck::grid_sort_waves(M) * (int64_t)sizeof(uint32_t);
    return ck::ck_sort_passes(ck::ck_key_bits(E)) > 1 ? 4 * M * (int64_t)sizeof(uint32_t) : 0;
}

// The launches of ck_moe_sort; `workspace` holds ck_moe_sort_workspace_size(M, E) bytes (checked by the callers).
static int moe_sort_launch(const void* expert_ids, int ids_are_i32, int64_t* sorted_expert_idxs,
                           int64_t* sorted_scattered_idxs, int64_t* expert_offsets, void* workspace, int64_t M,
                           int64_t E, hipStream_t s) {
    const int key_bits = ck::ck_key_bits(E);
    if (use_grid_sort(M, E)) {
        if (reinterpret_cast<uintptr_t>(workspace) & 3u) return CK_ERR_WORKSPACE;
        const int num_waves = ck::grid_sort_waves(M);
        const unsigned grid = (unsigned)ck_ceil_div(num_waves, ck::kGridSortBlockWaves);
        uint32_t* hist = (uint32_t*)workspace;
        const int total = (1 << key_bits) * num_waves;
        ck::SortedStorer store = {sorted_expert_idxs, sorted_scattered_idxs};
        if (ids_are_i32) {
            ck::ExpertIdLoader<true> load = {expert_ids};
            hipLaunchKernelGGL(ck::moe_grid_hist_kernel<true>, dim3(grid), dim3(256), 0, s, load, (int)M, key_bits, hist,
                               num_waves);
            hipLaunchKernelGGL(ck::moe_grid_scan_kernel, dim3(1), dim3(1024), 0, s, hist, total);
            hipLaunchKernelGGL(ck::moe_grid_scatter_kernel<true>, dim3(grid), dim3(256), 0, s, load, store, (int)M,
                               key_bits, hist, num_waves, expert_offsets, (int)E);
        } else {
            ck::ExpertIdLoader<false> load = {expert_ids};
            hipLaunchKernelGGL(ck::moe_grid_hist_kernel<false>, dim3(grid), dim3(256), 0, s, load, (int)M, key_bits, hist,
                               num_waves);
            hipLaunchKernelGGL(ck::moe_grid_scan_kernel, dim3(1), dim3(1024), 0, s, hist, total);
            hipLaunchKernelGGL(ck::moe_grid_scatter_kernel<false>, dim3(grid), dim3(256), 0, s, load, store, (int)M,
                               key_bits, hist, num_waves, expert_offsets, (int)E);
        }
        return ck_launch_status();
    }
    if (ids_are_i32)
        hipLaunchKernelGGL(ck::moe_sort_kernel<true>, dim3(1), dim3(ck::kSortThreads), 0, s, expert_ids,
                           sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, (uint32_t*)workspace, (int)M,
                           (int)E, key_bits);
    else
        hipLaunchKernelGGL(ck::moe_sort_kernel<false>, dim3(1), dim3(ck::kSortThreads), 0, s, expert_ids,
                           sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, (uint32_t*)workspace, (int)M,
                           (int)E, key_bits);
    return ck_launch_status();
}

static int moe_sort_check(const void* expert_ids, const int64_t* sorted_expert_idxs,
                          const int64_t* sorted_scattered_idxs, const int64_t* expert_offsets, int64_t M, int64_t E) {
    if (M < 0 || E <= 0 || M > 0x7fffffff || E > 0x7fffffff) return CK_ERR_SHAPE;
    if (!expert_offsets) return CK_ERR_NULL;
    if (M > 0 && (!expert_ids || !sorted_expert_idxs || !sorted_scattered_idxs)) return CK_ERR_NULL;
    return CK_OK;
}

extern "C" int ck_moe_sort(const void* expert_ids, int ids_are_i32, int64_t* sorted_expert_idxs,
                           int64_t* sorted_scattered_idxs, int64_t* expert_offsets, void* workspace,
                           int64_t workspace_bytes, int64_t M, int64_t E, void* stream) {
    const int bad = moe_sort_check(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, M, E);
    if (bad) return bad;
    const int64_t need = ck_moe_sort_workspace_size(M, E);
    if (need > 0 && (!workspace || workspace_bytes < need)) return CK_ERR_WORKSPACE;
    return moe_sort_launch(expert_ids, ids_are_i32, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                           workspace, M, E, (hipStream_t)stream);
}

// ---- the same sort for callers that cannot allocate -----------------------------------------------
// The workspace of ck_moe_sort (the grid-wide sort's [bins][waves] histogram, or the key / value ping-pong
// arrays of a multi-pass single-workgroup sort) lives in this file-scope device array instead of a buffer the
// caller brings.  Every GPU the library runs on holds its own copy until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress: the kernels get the address that call returns for
// the current device, kept per device below.  Nothing in it has to start at zero (the histogram kernel writes
// every entry the scan reads, a radix pass writes every pair the next one reads), so no clearing is needed;
// two calls that overlap on one GPU (different streams) would share it and race.
static __device__ __align__(256) unsigned char scratch[CK_MOE_SORT_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int scratch_for_current_device(void** out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return CK_ERR_RUNTIME;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return CK_ERR_RUNTIME;
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return CK_OK;
}
}  // namespace

extern "C" int ck_moe_sort_noalloc(const void* expert_ids, int ids_are_i32, int64_t* sorted_expert_idxs,
                                   int64_t* sorted_scattered_idxs, int64_t* expert_offsets, int64_t M, int64_t E,
                                   void* stream) {
    const int bad = moe_sort_check(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, M, E);
    if (bad) return bad;
    if (ck_moe_sort_workspace_size(M, E) > (int64_t)CK_MOE_SORT_NOALLOC_SCRATCH_BYTES) return CK_ERR_SCRATCH;
    void* ptr = nullptr;
    const int status = scratch_for_current_device(&ptr);
    if (status) return status;
    return moe_sort_launch(expert_ids, ids_are_i32, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, ptr, M,
                           E, (hipStream_t)stream);
}

extern "C" int ck_offsets_from_sorted(const int64_t* sorted_expert_idxs, int64_t* expert_offsets, int64_t M, int64_t E,
                                      void* stream) {
    if (M < 0 || E <= 0) return CK_ERR_SHAPE;
    if (!expert_offsets || (M > 0 && !sorted_expert_idxs)) return CK_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    int64_t blocks = ck_ceil_div(M > E ? M : E, 256);
    if (blocks > 1024) blocks = 1024;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(ck::offsets_from_sorted_kernel, dim3((unsigned)blocks), dim3(256), 0, s, sorted_expert_idxs,
                       expert_offsets, M, E);
    return ck_launch_status();
}
