// Element-wise additions for gfx950: output = x + y (two tensors) and output = x + scalar.
// Take the place of cute_kernels/kernels/add/add_tensor/cuda_implementation/kernels_forward.cu and
// cute_kernels/kernels/add/add_scalar/cuda_implementation/kernels_forward.cu.  HBM-bound streaming
// kernels like the SwiGLU ones: 16-byte non-temporal packets, several per lane in flight, the sum
// formed in fp32 and rounded once (which is what `x + y` gives on stock torch for every storage type).
// One instantiation for 16-byte packets and one for single elements (unaligned pointers).
#include "ck_device.h"

namespace ck {

constexpr int kAddUnroll = 4;  // packets per lane

// SCALAR: y is ignored and `addend` is added to every element
template <typename T, int VEC, bool SCALAR>
__global__ void add_kernel(const typename T::storage_t* __restrict__ x, const typename T::storage_t* __restrict__ y,
                           float addend, typename T::storage_t* __restrict__ out, int64_t num_elements) {
    typedef VPack<T, VEC> P;
    const int64_t num_packs = num_elements / VEC;
    const int64_t base = (int64_t)blockIdx.x * blockDim.x * kAddUnroll + threadIdx.x;
    P a[kAddUnroll], b[kAddUnroll];
#pragma unroll
    for (int i = 0; i < kAddUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            a[i] = nt_load(reinterpret_cast<const P*>(x) + p);
            if (!SCALAR) b[i] = nt_load(reinterpret_cast<const P*>(y) + p);
        }
    }
#pragma unroll
    for (int i = 0; i < kAddUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            P o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o.v[j] = T::down(T::up(a[i].v[j]) + (SCALAR ? addend : T::up(b[i].v[j])));
            nt_store(o, reinterpret_cast<P*>(out) + p);
        }
    }
    // the last (num_elements % VEC) scalars: first lanes of block 0
    if (VEC > 1 && blockIdx.x == 0) {
        const int64_t e = num_packs * VEC + threadIdx.x;
        if (e < num_elements) out[e] = T::down(T::up(x[e]) + (SCALAR ? addend : T::up(y[e])));
    }
}

}  // namespace ck

namespace {

bool valid_block(int block_size) { return block_size >= 64 && block_size <= 1024 && block_size % 64 == 0; }

template <bool SCALAR>
int launch_add(const void* x, const void* y, float addend, void* output, int64_t num_elements, int dtype, int block_size,
               void* stream) {
    if (num_elements < 0 || !valid_block(block_size)) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (num_elements == 0) return CK_OK;
    if (!x || !output || (!SCALAR && !y)) return CK_ERR_NULL;
    if (!ck_aligned_elem(x, dtype) || !ck_aligned_elem(output, dtype) || (!SCALAR && !ck_aligned_elem(y, dtype)))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = ck_aligned16(x) && ck_aligned16(output) && (SCALAR || ck_aligned16(y));
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const int64_t items = vec ? num_elements / T::kVec : num_elements;
        const int64_t g = items <= 0 ? 1 : ck_ceil_div(items, (int64_t)block_size * ck::kAddUnroll);
        if (g > 0x7fffffff) return CK_ERR_SHAPE;
        if (vec)
            hipLaunchKernelGGL((ck::add_kernel<T, T::kVec, SCALAR>), dim3((unsigned)g), dim3(block_size), 0, s,
                               (const S*)x, (const S*)y, addend, (S*)output, num_elements);
        else
            hipLaunchKernelGGL((ck::add_kernel<T, 1, SCALAR>), dim3((unsigned)g), dim3(block_size), 0, s, (const S*)x,
                               (const S*)y, addend, (S*)output, num_elements);
    });
    return ck_launch_status();
}

}  // namespace

extern "C" int ck_add_tensor_forward(const void* x, const void* y, void* output, int64_t num_elements, int dtype,
                                     int block_size, void* stream) {
    return launch_add<false>(x, y, 0.f, output, num_elements, dtype, block_size, stream);
}

extern "C" int ck_add_scalar_forward(const void* x, double y, void* output, int64_t num_elements, int dtype,
                                     int block_size, void* stream) {
    return launch_add<true>(x, nullptr, (float)y, output, num_elements, dtype, block_size, stream);
}
