// Routing weights of the MoE layer in one pass: the k largest router logits of every token, their positions, and
// the softmax over those k values.  The reference does this with stock torch ops - topk (or max for k = 1), a cast
// to fp32, softmax, a cast back (cute_kernels/kernels/scattermoe/torch_implementation.py:121-132, 193-199) - and
// autograd strings the matching backward ops together; here each direction is one launch, one wavefront per token.
//   forward : selected[t, j]  = position of the j-th largest logit of token t (ties: the lower position first;
//                               NaN counts as larger than every number, as in torch.topk)
//             weights[t, j]   = exp(v_j - v_0) / sum_i exp(v_i - v_0) over the k selected values, fp32 math,
//                               rounded once to the storage type; the fp32 values are kept for the backward
//   backward: d_v[t, j]       = w_j * (g_j - sum_i g_i w_i)     (softmax backward on the fp32 weights)
//             d_logits[t, e]  = d_v[t, j] where e = selected[t, j], else 0  (every element of the row is written)
#include <math.h>

#include "ck_device.h"

namespace ck {

// is (a, ai) ahead of (b, bi) in the order "larger value first, NaN before everything, lower position first"?
__device__ __forceinline__ bool router_ahead(float a, int ai, float b, int bi) {
    const bool an = a != a, bn = b != b;
    const bool gt = (a > b) || (an && !bn);
    const bool eq = (a == b) || (an && bn);
    return gt || (eq && ai < bi);
}

template <typename T, int VPL>
__global__ void __launch_bounds__(256)
    router_fwd_kernel(const typename T::storage_t* __restrict__ logits, int64_t ld,
                      typename T::storage_t* __restrict__ weights, float* __restrict__ weights_f32,
                      int64_t* __restrict__ selected, int64_t tokens, int E, int k) {
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    float v[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = i * CK_WAVE + lane;
        v[i] = e < E ? T::up(logits[t * ld + e]) : 0.f;
    }
    uint32_t taken = 0;  // bit i: v[i] is already among the selected
    float my_val = 0.f;  // lane j < k ends up with the j-th largest value and its position
    int my_idx = 0;
    for (int j = 0; j < k; ++j) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int e = i * CK_WAVE + lane;
            if (e < E && !((taken >> i) & 1u) && router_ahead(v[i], e, best, bi)) {
                best = v[i];
                bi = e;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(best, off, CK_WAVE);
            const int oi = __shfl_xor(bi, off, CK_WAVE);
            if (router_ahead(ov, oi, best, bi)) {
                best = ov;
                bi = oi;
            }
        }
        if (lane == j) {
            my_val = best;
            my_idx = bi;
        }
        if ((bi % CK_WAVE) == lane) taken |= 1u << (bi / CK_WAVE);
    }
    const float top = __shfl(my_val, 0, CK_WAVE);
    const float p = lane < k ? expf(my_val - top) : 0.f;
    const float w = p / wave_sum(p);
    if (lane < k) {
        weights[t * k + lane] = T::down(w);
        weights_f32[t * k + lane] = w;
        selected[t * k + lane] = my_idx;
    }
}

template <typename T, int VPL>
__global__ void __launch_bounds__(256)
    router_bwd_kernel(const typename T::storage_t* __restrict__ d_weights, const float* __restrict__ weights_f32,
                      const int64_t* __restrict__ selected, typename T::storage_t* __restrict__ d_logits, int64_t ld,
                      int64_t tokens, int E, int k) {
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    const bool live = lane < k;
    const float w = live ? weights_f32[t * k + lane] : 0.f;
    const float g = live ? T::up(d_weights[t * k + lane]) : 0.f;
    const int sel = live ? (int)selected[t * k + lane] : -1;
    const float dv = w * (g - wave_sum(g * w));
    float out[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) out[i] = 0.f;
    for (int j = 0; j < k; ++j) {
        const int sj = __shfl(sel, j, CK_WAVE);
        const float dj = __shfl(dv, j, CK_WAVE);
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (i * CK_WAVE + lane == sj) out[i] = dj;
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = i * CK_WAVE + lane;
        if (e < E) d_logits[t * ld + e] = T::down(out[i]);
    }
}

}  // namespace ck

namespace {
constexpr int64_t kMaxRouterExperts = 1024;  // 16 values per lane
}

#define CK_ROUTER_LAUNCH(KERNEL, ...)                                                                              \
    do {                                                                                                           \
        const int vpl = (int)ck_ceil_div(E, (int64_t)CK_WAVE);                                                     \
        if (vpl <= 1)                                                                                              \
            hipLaunchKernelGGL((ck::KERNEL<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 2)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 2>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 4)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 4>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 8)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 8>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else                                                                                                       \
            hipLaunchKernelGGL((ck::KERNEL<T, 16>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);           \
    } while (0)

extern "C" int ck_router_topk_softmax_forward(const void* logits, int64_t logits_stride, void* weights,
                                              float* weights_f32, int64_t* selected, int64_t tokens, int64_t E,
                                              int64_t k, int dtype, void* stream) {
    if (tokens < 0 || E <= 0 || E > kMaxRouterExperts || k <= 0 || k > E || k > CK_WAVE || logits_stride < E)
        return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!logits || !weights || !weights_f32 || !selected) return CK_ERR_NULL;
    if (!ck_aligned_elem(logits, dtype) || !ck_aligned_elem(weights, dtype)) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        CK_ROUTER_LAUNCH(router_fwd_kernel, (const S*)logits, logits_stride, (S*)weights, weights_f32, selected, tokens,
                         (int)E, (int)k);
    });
    return ck_launch_status();
}

extern "C" int ck_router_topk_softmax_backward(const void* d_weights, const float* weights_f32, const int64_t* selected,
                                               void* d_logits, int64_t d_logits_stride, int64_t tokens, int64_t E,
                                               int64_t k, int dtype, void* stream) {
    if (tokens < 0 || E <= 0 || E > kMaxRouterExperts || k <= 0 || k > E || k > CK_WAVE || d_logits_stride < E)
        return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!d_weights || !weights_f32 || !selected || !d_logits) return CK_ERR_NULL;
    if (!ck_aligned_elem(d_weights, dtype) || !ck_aligned_elem(d_logits, dtype)) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        CK_ROUTER_LAUNCH(router_bwd_kernel, (const S*)d_weights, weights_f32, selected, (S*)d_logits, d_logits_stride,
                         tokens, (int)E, (int)k);
    });
    return ck_launch_status();
}
