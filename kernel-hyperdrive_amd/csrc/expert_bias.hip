// Per-expert bias of the grouped linears, and its gradient.
// The reference's plain-torch experts apply it as F.linear(rows_e, W[e], bias[e])
// (cute_kernels/kernels/scattermoe/torch_implementation.py:35-43); its Triton experts never read the parameter
// (triton_implementation/__init__.py:24-34).  Here the bias is a pass over the grouped product's output:
//   forward : y[r(i), :] += bias[e(i), :]                 i = position in expert-sorted order, e(i) its expert,
//                                                         r(i) = row_index ? row_index[i] : i
//   backward: d_bias[e, :] = sum_{i in expert e} dy[i, :]  over expert-grouped rows, fp32 sum, one rounding
// Both are HBM-bound: the forward reads and writes y once, the backward reads dy once.
#include "ck_device.h"

namespace ck {

// expert owning sorted position i: the first e with offsets[e] > i (offsets are inclusive running totals)
__device__ inline int expert_of_position(const int64_t* __restrict__ offsets, int E, int64_t i) {
    int lo = 0, hi = E - 1;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (offsets[mid] > i)
            hi = mid;
        else
            lo = mid + 1;
    }
    return lo;
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    expert_bias_fwd_kernel(typename T::storage_t* __restrict__ y, int64_t ld_y,
                           const typename T::storage_t* __restrict__ bias, int64_t ld_bias,
                           const int64_t* __restrict__ row_index, const int64_t* __restrict__ offsets, int64_t M,
                           int64_t N, int E) {
    typedef VPack<T, VEC> P;
    const int64_t i = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (i >= M) return;
    const int lane = lane_id();
    const int e = expert_of_position(offsets, E, i);
    const int64_t r = row_index != nullptr ? row_index[i] : i;
    P* row = reinterpret_cast<P*>(y + r * ld_y);
    const P* b = reinterpret_cast<const P*>(bias + (int64_t)e * ld_bias);
    const int64_t packs = N / VEC;
    for (int64_t p = lane; p < packs; p += CK_WAVE) {
        P v = nt_load(row + p);
        const P bv = b[p];
#pragma unroll
        for (int j = 0; j < VEC; ++j) v.v[j] = T::down(T::up(v.v[j]) + T::up(bv.v[j]));
        nt_store(v, row + p);
    }
}

// One workgroup per (column block of 64 * VEC, expert): four teams of 64 lanes walk the expert's rows
// interleaved, each lane summing VEC columns, and the teams' sums meet in LDS in a fixed order.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    expert_bias_bwd_kernel(const typename T::storage_t* __restrict__ dy, int64_t ld_dy,
                           const int64_t* __restrict__ offsets, typename T::storage_t* __restrict__ d_bias,
                           int64_t ld_dbias, int64_t N) {
    typedef VPack<T, VEC> P;
    __shared__ float part[3][CK_WAVE * VEC];
    const int e = blockIdx.y;
    const int team = threadIdx.x / CK_WAVE;
    const int lane = lane_id();
    const int64_t col = ((int64_t)blockIdx.x * CK_WAVE + lane) * VEC;
    const int64_t begin = e == 0 ? 0 : offsets[e - 1];
    const int64_t end = offsets[e];
    const bool live = col < N;  // N is a multiple of VEC on this path
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    if (live) {
        int64_t i = begin + team;
        // two rows in flight per team
        for (; i + 4 < end; i += 8) {
            const P a = nt_load(reinterpret_cast<const P*>(dy + i * ld_dy + col));
            const P b = nt_load(reinterpret_cast<const P*>(dy + (i + 4) * ld_dy + col));
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += T::up(a.v[j]);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += T::up(b.v[j]);
        }
        if (i < end) {
            const P a = nt_load(reinterpret_cast<const P*>(dy + i * ld_dy + col));
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += T::up(a.v[j]);
        }
    }
    if (team > 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) part[team - 1][lane * VEC + j] = acc[j];
    }
    __syncthreads();
    if (team == 0 && live) {
        P o;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            o.v[j] = T::down(((acc[j] + part[0][lane * VEC + j]) + part[1][lane * VEC + j]) + part[2][lane * VEC + j]);
        *reinterpret_cast<P*>(d_bias + (int64_t)e * ld_dbias + col) = o;
    }
}

}  // namespace ck

extern "C" int ck_expert_bias_forward(void* y, int64_t y_stride, const void* bias, int64_t bias_stride,
                                      const int64_t* row_index, const int64_t* expert_offsets, int64_t num_rows,
                                      int64_t N, int64_t E, int dtype, void* stream) {
    if (num_rows < 0 || N < 0 || E <= 0 || E > 0x7fffffff || y_stride < N || bias_stride < N) return CK_ERR_SHAPE;
    if (num_rows == 0 || N == 0) return CK_OK;
    if (!y || !bias || !expert_offsets) return CK_ERR_NULL;
    if (!ck_aligned_elem(y, dtype) || !ck_aligned_elem(bias, dtype)) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(num_rows, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(y) && ck_aligned16(bias) && N % T::kVec == 0 && y_stride % T::kVec == 0 &&
                         bias_stride % T::kVec == 0;
        if (vec)
            hipLaunchKernelGGL((ck::expert_bias_fwd_kernel<T, T::kVec>), dim3((unsigned)grid), dim3(256), 0, s, (S*)y,
                               y_stride, (const S*)bias, bias_stride, row_index, expert_offsets, num_rows, N, (int)E);
        else
            hipLaunchKernelGGL((ck::expert_bias_fwd_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, (S*)y, y_stride,
                               (const S*)bias, bias_stride, row_index, expert_offsets, num_rows, N, (int)E);
    });
    return ck_launch_status();
}

extern "C" int ck_expert_bias_backward(const void* dy, int64_t dy_stride, const int64_t* expert_offsets, void* d_bias,
                                       int64_t d_bias_stride, int64_t num_rows, int64_t N, int64_t E, int dtype,
                                       void* stream) {
    if (num_rows < 0 || N < 0 || E <= 0 || E > 65535 || dy_stride < N || d_bias_stride < N) return CK_ERR_SHAPE;
    if (N == 0) return CK_OK;
    if (!d_bias || !expert_offsets || (num_rows > 0 && !dy)) return CK_ERR_NULL;
    if (!ck_aligned_elem(dy, dtype) || !ck_aligned_elem(d_bias, dtype)) return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(dy) && ck_aligned16(d_bias) && N % T::kVec == 0 && dy_stride % T::kVec == 0 &&
                         d_bias_stride % T::kVec == 0;
        if (vec) {
            const int64_t blocks = ck_ceil_div(N, (int64_t)CK_WAVE * T::kVec);
            if (blocks > 0x7fffffff) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::expert_bias_bwd_kernel<T, T::kVec>), dim3((unsigned)blocks, (unsigned)E), dim3(256), 0,
                               s, (const S*)dy, dy_stride, expert_offsets, (S*)d_bias, d_bias_stride, N);
        } else {
            const int64_t blocks = ck_ceil_div(N, (int64_t)CK_WAVE);
            if (blocks > 0x7fffffff) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::expert_bias_bwd_kernel<T, 1>), dim3((unsigned)blocks, (unsigned)E), dim3(256), 0, s,
                               (const S*)dy, dy_stride, expert_offsets, (S*)d_bias, d_bias_stride, N);
        }
    });
    return ck_launch_status();
}
