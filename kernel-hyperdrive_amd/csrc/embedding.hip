// Embedding gather (forward) and scatter-add (backward) for gfx950.
//   forward : out[i, :] = W[ids[i], :]                    bit-exact row copy
//             (cute_kernels/kernels/embedding/triton_implementation/kernels_forward.py:13-39)
//   backward: dW = one_hot(ids)^T @ dy  with fp32 accumulation and ONE rounding per element
//             (math: cute_kernels/kernels/embedding/README.md:7-15).  The reference adds rows with
//             floating-point atomics into a zeroed table (kernels_backward.py:13-45); here the token
//             ids are sorted first so that every table row has exactly one writer:
//               1. sort kernel (one workgroup): stable radix sort of (id, position); marks which
//                  table rows are selected at all; for every sorted slot the index of the first slot
//                  of its run of equal ids.
//               2. fill kernel: rows no id selects are written as zeros (the bulk of the traffic).
//               3. chunk kernel: a run of equal ids is cut into chunks of kChunk slots; one wave sums
//                  the dy rows of a chunk in fp32 registers, in ascending token position.  A run that
//                  fits one chunk is rounded and stored straight into dW; longer runs leave one fp32
//                  partial row per chunk in the workspace.
//               4. combine kernel: sums the partial rows of each long run and stores the dW row.
//             No floating-point atomics, no zero-fill of rows that are written anyway, deterministic.
#include "ck_block_sort.h"

namespace ck {

constexpr int kChunk = 32;      // slots of one run summed by one wave
constexpr int kRowPacks = 8;    // packets per lane per column tile (tile = 64 lanes * 8 packets)

// accumulator of the backward sums
template <typename T>
struct AccOf {
    typedef float type;
};
template <>
struct AccOf<F32> {
    typedef double type;
};

template <bool I32>
__device__ __forceinline__ int64_t load_tok(const void* p, int64_t i) {
    return I32 ? (int64_t) reinterpret_cast<const int32_t*>(p)[i] : reinterpret_cast<const int64_t*>(p)[i];
}

// ---- forward ---------------------------------------------------------------------------------
// One wave per output row, 4 rows per workgroup.  VEC = T::kVec (16-byte packets) or 1.
template <typename T, int VEC, bool I32>
__global__ void __launch_bounds__(256)
    embedding_fwd_kernel(const void* __restrict__ ids, const typename T::storage_t* __restrict__ w,
                         typename T::storage_t* __restrict__ out, int64_t n, int64_t V, int64_t H) {
    typedef VPack<T, VEC> P;
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (row >= n) return;
    const int lane = lane_id();
    const int64_t id = load_tok<I32>(ids, row);
    const int64_t packs = H / VEC;
    P* dst = reinterpret_cast<P*>(out + row * H);
    if (id < 0 || id >= V) {
        P z;
#pragma unroll
        for (int j = 0; j < VEC; ++j) z.v[j] = T::down(0.f);
        for (int64_t p = lane; p < packs; p += CK_WAVE) dst[p] = z;
        return;
    }
    const P* src = reinterpret_cast<const P*>(w + id * H);
    int64_t p = lane;
    // four packets in flight per lane
    for (; p + 3 * CK_WAVE < packs; p += 4 * CK_WAVE) {
        const P a = src[p], b = src[p + CK_WAVE], c = src[p + 2 * CK_WAVE], d = src[p + 3 * CK_WAVE];
        nt_store(a, dst + p);
        nt_store(b, dst + p + CK_WAVE);
        nt_store(c, dst + p + 2 * CK_WAVE);
        nt_store(d, dst + p + 3 * CK_WAVE);
    }
    for (; p < packs; p += CK_WAVE) nt_store(src[p], dst + p);
}

// ---- backward 1: sort -------------------------------------------------------------------------
struct EmbWorkspace {
    uint32_t* keys[2];
    uint32_t* vals[2];
    uint32_t* run_head;  // [n] first sorted slot of the run of equal ids that slot i belongs to
    uint8_t* touched;    // [V] 1 when some id selects the row
    float* partial;      // [2 * ceil(n / kChunk)][H]
};

static inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static inline int64_t emb_carve(void* base, int64_t n, int64_t V, int64_t H, EmbWorkspace* ws) {
    int64_t off = 0;
    char* b = (char*)base;
    const int64_t arr = align_up(n * 4, 256);
    for (int i = 0; i < 2; ++i) {
        if (ws) ws->keys[i] = (uint32_t*)(b + off);
        off += arr;
        if (ws) ws->vals[i] = (uint32_t*)(b + off);
        off += arr;
    }
    if (ws) ws->run_head = (uint32_t*)(b + off);
    off += arr;
    if (ws) ws->touched = (uint8_t*)(b + off);
    off += align_up(V, 256);
    if (ws) ws->partial = (float*)(b + off);
    off += align_up(2 * ((n + kChunk - 1) / kChunk) * H * 4, 256);
    return off;
}

template <bool I32>
__global__ void __launch_bounds__(kSortThreads)
    embedding_sort_kernel(const void* __restrict__ ids, EmbWorkspace ws, int n, int64_t V, int key_bits) {
    __shared__ SortShared sh;
    __shared__ int wave_last[kSortWaves];

    // clear the row marks (V bytes, padded to a multiple of 256 by the workspace layout)
    uint32_t* tw = reinterpret_cast<uint32_t*>(ws.touched);
    for (int64_t i = threadIdx.x; i < (V + 3) / 4; i += kSortThreads) tw[i] = 0u;

    const int passes = ck_sort_passes(key_bits);
    const int bits_per_pass = (key_bits + passes - 1) / passes;
    for (int p = 0; p < passes; ++p) {
        const int shift = p * bits_per_pass;
        const int bits = min(bits_per_pass, key_bits - shift);
        const bool first = p == 0;
        const uint32_t* kin = ws.keys[(p + 1) & 1];
        const uint32_t* vin = ws.vals[(p + 1) & 1];
        uint32_t* kout = ws.keys[p & 1];
        uint32_t* vout = ws.vals[p & 1];
        auto load = [&](int i, uint32_t& k, uint32_t& v) {
            if (first) {
                const int64_t id = load_tok<I32>(ids, i);
                k = (id < 0 || id >= V) ? (uint32_t)V : (uint32_t)id;  // invalid ids sort last and are skipped
                v = (uint32_t)i;
            } else {
                k = kin[i];
                v = vin[i];
            }
        };
        auto store = [&](int pos, uint32_t k, uint32_t v) {
            kout[pos] = k;
            vout[pos] = v;
        };
        block_radix_pass(sh, n, shift, bits, load, store);
    }
    const uint32_t* skeys = ws.keys[(passes - 1) & 1];

    // run heads: each lane owns a contiguous range of sorted slots; the index of the last head at or
    // before a slot is a running maximum, carried across lanes with a wave scan and across waves in LDS
    const int per = (n + kSortThreads - 1) / kSortThreads;
    const int b0 = min((int)threadIdx.x * per, n);
    const int b1 = min(b0 + per, n);
    int last = -1;
    for (int i = b0; i < b1; ++i) {
        const uint32_t k = skeys[i];
        if (i == 0 || skeys[i - 1] != k) {
            last = i;
            if ((int64_t)k < V) ws.touched[k] = 1;
        }
    }
    const int wave = threadIdx.x / CK_WAVE;
    const int incl = wave_inclusive_max_i(last);
    if (lane_id() == CK_WAVE - 1) wave_last[wave] = incl;
    __syncthreads();
    int carry = __shfl_up(incl, 1, CK_WAVE);
    if (lane_id() == 0) carry = -1;
    for (int w = 0; w < wave; ++w) carry = max(carry, wave_last[w]);
    for (int i = b0; i < b1; ++i) {
        if (i == 0 || skeys[i - 1] != skeys[i]) carry = i;
        ws.run_head[i] = (uint32_t)carry;
    }
}

// ---- backward 2: zero rows nobody selects ---------------------------------------------------------
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    embedding_bwd_fill_kernel(const uint8_t* __restrict__ touched, typename T::storage_t* __restrict__ dw, int64_t V,
                              int64_t H) {
    typedef VPack<T, VEC> P;
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (row >= V) return;
    if (touched[row]) return;
    P z;
#pragma unroll
    for (int j = 0; j < VEC; ++j) z.v[j] = T::down(0.f);
    P* dst = reinterpret_cast<P*>(dw + row * H);
    const int64_t packs = H / VEC;
    for (int64_t p = lane_id(); p < packs; p += CK_WAVE) nt_store(z, dst + p);
}

// ---- backward 3: sum the dy rows of one chunk of a run ----------------------------------------------
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    embedding_bwd_chunk_kernel(const uint32_t* __restrict__ skeys, const uint32_t* __restrict__ spos,
                               const uint32_t* __restrict__ run_head, const typename T::storage_t* __restrict__ dy,
                               typename T::storage_t* __restrict__ dw, float* __restrict__ partial, int n, int64_t V,
                               int64_t H) {
    typedef VPack<T, VEC> P;
    const int i = blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (i >= n) return;
    const uint32_t id = skeys[i];
    if ((int64_t)id >= V) return;
    const int head = (int)run_head[i];
    if ((i - head) % kChunk != 0) return;
    const int lane = lane_id();

    // slots of this chunk: leading slots i, i+1, ... with the same id, at most kChunk
    const bool same = lane < kChunk && i + lane < n && skeys[i + lane] == id;
    const uint64_t bal = __ballot(same);
    const int cnt = __ffsll((unsigned long long)~bal) - 1;  // lane 0 always matches, so cnt >= 1
    const bool continues = cnt == kChunk && i + kChunk < n && skeys[i + kChunk] == id;
    const bool multi = (i != head) || continues;
    const uint32_t my_pos = lane < cnt ? spos[i + lane] : 0u;

    const int64_t packs = H / VEC;
    const int64_t tile = (int64_t)CK_WAVE * kRowPacks;
    // fp32 tables sum in fp64 so that the result is the correctly rounded sum whatever the order
    typedef typename AccOf<T>::type acc_t;
    for (int64_t p0 = 0; p0 < packs; p0 += tile) {
        acc_t acc[kRowPacks][VEC];
#pragma unroll
        for (int q = 0; q < kRowPacks; ++q)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[q][j] = 0;
        for (int r = 0; r < cnt; ++r) {
            const uint32_t pos = __shfl(my_pos, r, CK_WAVE);
            const P* src = reinterpret_cast<const P*>(dy + (int64_t)pos * H);
            P v[kRowPacks];
#pragma unroll
            for (int q = 0; q < kRowPacks; ++q) {
                const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                if (p < packs) v[q] = nt_load(src + p);
            }
#pragma unroll
            for (int q = 0; q < kRowPacks; ++q) {
                const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                if (p < packs) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[q][j] += (acc_t)T::up(v[q].v[j]);
                }
            }
        }
        if (!multi) {
            P* dst = reinterpret_cast<P*>(dw + (int64_t)id * H);
#pragma unroll
            for (int q = 0; q < kRowPacks; ++q) {
                const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                if (p < packs) {
                    P o;
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o.v[j] = T::down((float)acc[q][j]);
                    nt_store(o, dst + p);
                }
            }
        } else {
            // at most two chunk starts of long runs fall into one window of kChunk slots: the last chunk
            // of one run and the head of the next, told apart by the low bit
            const int64_t slot = 2 * (int64_t)(i / kChunk) + (i == head ? 1 : 0);
            float* dst = partial + slot * H;
#pragma unroll
            for (int q = 0; q < kRowPacks; ++q) {
                const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                if (p < packs) {
                    if (VEC % 4 == 0) {
#pragma unroll
                        for (int j = 0; j + 3 < VEC; j += 4)
                            *reinterpret_cast<float4*>(dst + p * VEC + j) = make_float4(
                                (float)acc[q][j], (float)acc[q][j + 1], (float)acc[q][j + 2], (float)acc[q][j + 3]);
                    } else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) dst[p * VEC + j] = (float)acc[q][j];
                    }
                }
            }
        }
    }
}

// ---- backward 4: add up the partial rows of long runs --------------------------------------------
// One workgroup per sorted slot; only heads of runs longer than kChunk do work.  Lane per column.
template <typename T>
__global__ void __launch_bounds__(256)
    embedding_bwd_combine_kernel(const uint32_t* __restrict__ skeys, const uint32_t* __restrict__ run_head,
                                 const float* __restrict__ partial, typename T::storage_t* __restrict__ dw, int n,
                                 int64_t V, int64_t H) {
    const int i = blockIdx.x;
    const uint32_t id = skeys[i];
    if ((int64_t)id >= V) return;
    if ((int)run_head[i] != i) return;
    if (!(i + kChunk < n && skeys[i + kChunk] == id)) return;
    typedef typename AccOf<T>::type acc_t;
    for (int64_t c = threadIdx.x; c < H; c += blockDim.x) {
        acc_t acc = 0;
        for (int s = i; s < n && skeys[s] == id; s += kChunk) {
            const int64_t slot = 2 * (int64_t)(s / kChunk) + (s == i ? 1 : 0);
            acc += (acc_t)partial[slot * H + c];
        }
        dw[(int64_t)id * H + c] = T::down((float)acc);
    }
}

}  // namespace ck

template <typename T, int VEC, bool I32>
static void launch_fwd(unsigned grid, hipStream_t s, const void* ids, const void* weight, void* output, int64_t n,
                       int64_t V, int64_t H) {
    typedef typename T::storage_t S;
    hipLaunchKernelGGL((ck::embedding_fwd_kernel<T, VEC, I32>), dim3(grid), dim3(256), 0, s, ids, (const S*)weight,
                       (S*)output, n, V, H);
}

extern "C" int ck_embedding_forward(const void* ids, int ids_are_i32, const void* weight, void* output,
                                    int64_t num_ids, int64_t V, int64_t H, int dtype, void* stream) {
    if (num_ids < 0 || V < 0 || H < 0) return CK_ERR_SHAPE;
    if (num_ids == 0 || H == 0) return CK_OK;
    if (!ids || !output || (V > 0 && !weight)) return CK_ERR_NULL;
    if (!ck_aligned_elem(output, dtype) || (weight && !ck_aligned_elem(weight, dtype))) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(num_ids, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        const bool vec = ck_aligned16(weight) && ck_aligned16(output) && (H % T::kVec == 0);
        if (vec) {
            if (ids_are_i32) launch_fwd<T, T::kVec, true>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
            else launch_fwd<T, T::kVec, false>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
        } else {
            if (ids_are_i32) launch_fwd<T, 1, true>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
            else launch_fwd<T, 1, false>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
        }
    });
    return ck_launch_status();
}

extern "C" int64_t ck_embedding_backward_workspace_size(int64_t num_ids, int64_t V, int64_t H) {
    if (num_ids < 0 || V < 0 || H < 0) return 0;
    return ck::emb_carve(nullptr, num_ids, V, H, nullptr);
}

template <typename T, int VEC>
static void launch_bwd(hipStream_t s, const ck::EmbWorkspace& ws, int passes, const void* dy, void* dw, int n,
                       int64_t V, int64_t H) {
    typedef typename T::storage_t S;
    const uint32_t* skeys = ws.keys[(passes - 1) & 1];
    const uint32_t* spos = ws.vals[(passes - 1) & 1];
    hipLaunchKernelGGL((ck::embedding_bwd_fill_kernel<T, VEC>), dim3((unsigned)ck_ceil_div(V, 4)), dim3(256), 0, s,
                       ws.touched, (S*)dw, V, H);
    if (n > 0) {
        hipLaunchKernelGGL((ck::embedding_bwd_chunk_kernel<T, VEC>), dim3((unsigned)ck_ceil_div(n, 4)), dim3(256), 0, s,
                           skeys, spos, ws.run_head, (const S*)dy, (S*)dw, ws.partial, n, V, H);
        hipLaunchKernelGGL((ck::embedding_bwd_combine_kernel<T>), dim3((unsigned)n), dim3(256), 0, s, skeys,
                           ws.run_head, ws.partial, (S*)dw, n, V, H);
    }
}

extern "C" int ck_embedding_backward(const void* ids, int ids_are_i32, const void* output_grad, void* weight_grad,
                                     void* workspace, int64_t workspace_bytes, int64_t num_ids, int64_t V, int64_t H,
                                     int dtype, void* stream) {
    if (num_ids < 0 || V < 0 || H < 0 || num_ids > 0x7fffffff || V >= 0xffffffffll) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (V == 0 || H == 0) return CK_OK;
    if (!weight_grad || (num_ids > 0 && (!ids || !output_grad))) return CK_ERR_NULL;
    if (!ck_aligned_elem(weight_grad, dtype) || (output_grad && !ck_aligned_elem(output_grad, dtype)))
        return CK_ERR_ALIGN;
    if (ck_ceil_div(V, 4) > 0x7fffffff) return CK_ERR_SHAPE;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CK_ERR_WORKSPACE;
    if (workspace_bytes < ck_embedding_backward_workspace_size(num_ids, V, H)) return CK_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    ck::EmbWorkspace ws;
    ck::emb_carve(workspace, num_ids, V, H, &ws);
    const int key_bits = ck::ck_key_bits(V + 1);  // one extra key value marks ids outside [0, V)
    const int passes = ck::ck_sort_passes(key_bits);
    if (ids_are_i32)
        hipLaunchKernelGGL(ck::embedding_sort_kernel<true>, dim3(1), dim3(ck::kSortThreads), 0, s, ids, ws,
                           (int)num_ids, V, key_bits);
    else
        hipLaunchKernelGGL(ck::embedding_sort_kernel<false>, dim3(1), dim3(ck::kSortThreads), 0, s, ids, ws,
                           (int)num_ids, V, key_bits);
    CK_DISPATCH_DTYPE(dtype, {
        const bool vec = ck_aligned16(weight_grad) && (!output_grad || ck_aligned16(output_grad)) && (H % T::kVec == 0);
        if (vec) launch_bwd<T, T::kVec>(s, ws, passes, output_grad, weight_grad, (int)num_ids, V, H);
        else launch_bwd<T, 1>(s, ws, passes, output_grad, weight_grad, (int)num_ids, V, H);
    });
    return ck_launch_status();
}
