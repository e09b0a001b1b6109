// Mixing of a token's k expert outputs with its routing weights, and the gradient of those weights.
// The reference does both with torch.bmm on [T, 1, k] x [T, k, H] batches
// (cute_kernels/kernels/scattermoe/triton_implementation/ops.py:160-164 and :204), which turns into
// thousands of degenerate GEMMs; here each is one HBM-bound pass, one wavefront per token.
//   forward : out[t, :]      = sum_j gates[t, j] * expanded[t, j, :]      (gates == NULL: plain sum over j, the
//                              reference's `.view(T, k, H).sum(-2)` of ops.py:261)
//   backward: d_gates[t, j]  = sum_h expanded[t, j, h] * grad_out[t, h]
// fp32 accumulation, one rounding.
#include "ck_device.h"

namespace ck {

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    combine_fwd_kernel(const typename T::storage_t* __restrict__ expanded, const typename T::storage_t* __restrict__ gates,
                       typename T::storage_t* __restrict__ out, int64_t tokens, int k, int64_t H) {
    typedef VPack<T, VEC> P;
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    const int64_t packs = H / VEC;
    const P* src = reinterpret_cast<const P*>(expanded + t * k * H);
    P* dst = reinterpret_cast<P*>(out + t * H);
    for (int64_t p = lane; p < packs; p += CK_WAVE) {
        float acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
        for (int s = 0; s < k; ++s) {
            const float g = gates != nullptr ? T::up(gates[t * k + s]) : 1.0f;
            const P v = nt_load(src + (int64_t)s * packs + p);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += g * T::up(v.v[j]);
        }
        P o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o.v[j] = T::down(acc[j]);
        nt_store(o, dst + p);
    }
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    combine_bwd_gates_kernel(const typename T::storage_t* __restrict__ expanded,
                             const typename T::storage_t* __restrict__ grad_out, typename T::storage_t* __restrict__ d_gates,
                             int64_t tokens, int k, int64_t H) {
    typedef VPack<T, VEC> P;
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    const int64_t packs = H / VEC;
    const P* dy = reinterpret_cast<const P*>(grad_out + t * H);
    for (int s = 0; s < k; ++s) {
        const P* src = reinterpret_cast<const P*>(expanded + (t * k + s) * H);
        float acc = 0.f;
        for (int64_t p = lane; p < packs; p += CK_WAVE) {
            const P a = src[p];
            const P b = dy[p];  // re-read per slot: stays in L1 / L2
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc += T::up(a.v[j]) * T::up(b.v[j]);
        }
        acc = wave_sum(acc);
        if (lane == 0) d_gates[t * k + s] = T::down(acc);
    }
}

}  // namespace ck

extern "C" int ck_moe_combine_forward(const void* expanded, const void* gates, void* out, int64_t tokens, int64_t k,
                                      int64_t H, int dtype, void* stream) {
    if (tokens < 0 || k <= 0 || H < 0 || k > 0x7fffffff) return CK_ERR_SHAPE;
    if (tokens == 0 || H == 0) return CK_OK;
    if (!expanded || !out) return CK_ERR_NULL;
    if (!ck_aligned_elem(expanded, dtype) || (gates && !ck_aligned_elem(gates, dtype)) || !ck_aligned_elem(out, dtype))
        return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(expanded) && ck_aligned16(out) && H % T::kVec == 0;
        if (vec)
            hipLaunchKernelGGL((ck::combine_fwd_kernel<T, T::kVec>), dim3((unsigned)grid), dim3(256), 0, s,
                               (const S*)expanded, (const S*)gates, (S*)out, tokens, (int)k, H);
        else
            hipLaunchKernelGGL((ck::combine_fwd_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)expanded,
                               (const S*)gates, (S*)out, tokens, (int)k, H);
    });
    return ck_launch_status();
}

extern "C" int ck_moe_combine_backward_gates(const void* expanded, const void* grad_out, void* d_gates, int64_t tokens,
                                             int64_t k, int64_t H, int dtype, void* stream) {
    if (tokens < 0 || k <= 0 || H < 0 || k > 0x7fffffff) return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!d_gates || (H > 0 && (!expanded || !grad_out))) return CK_ERR_NULL;
    if (!ck_aligned_elem(expanded, dtype) || !ck_aligned_elem(grad_out, dtype) || !ck_aligned_elem(d_gates, dtype))
        return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(expanded) && ck_aligned16(grad_out) && H % T::kVec == 0;
        if (vec)
            hipLaunchKernelGGL((ck::combine_bwd_gates_kernel<T, T::kVec>), dim3((unsigned)grid), dim3(256), 0, s,
                               (const S*)expanded, (const S*)grad_out, (S*)d_gates, tokens, (int)k, H);
        else
            hipLaunchKernelGGL((ck::combine_bwd_gates_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, s,
                               (const S*)expanded, (const S*)grad_out, (S*)d_gates, tokens, (int)k, H);
    });
    return ck_launch_status();
}
