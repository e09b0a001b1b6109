// SwiGLU forward / backward for gfx950: y = up * gate * sigmoid(gate).
// HBM-bound streaming kernels: every lane moves 16-byte packets, several per lane in flight,
// fp32 math, one rounding on store.  Two forms:
//   - two-tensor form (gate, up separate), math of cute_kernels/kernels/swiglu/README.md:3-13;
//   - "unchunked" form on x[B, 2h] with up = x[:, :h], gate = x[:, h:]
//     (cute_kernels/kernels/swiglu_unchunked/torch_implementation.py:5-7).
// Every kernel is instantiated for packets of T::kVec elements (16 bytes) and, for pointers or row
// lengths that do not allow that, for packets of one element.
#include "ck_device.h"

namespace ck {

constexpr int kUnroll = 4;  // packets per lane per tensor

// ---- two-tensor form ---------------------------------------------------------------------
template <typename T, int VEC>
__global__ void swiglu_fwd_kernel(const typename T::storage_t* __restrict__ gate,
                                  const typename T::storage_t* __restrict__ up,
                                  typename T::storage_t* __restrict__ out, int64_t num_elements) {
    typedef VPack<T, VEC> P;
    const int64_t num_packs = num_elements / VEC;
    const int64_t base = (int64_t)blockIdx.x * blockDim.x * kUnroll + threadIdx.x;
    P g[kUnroll], u[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            g[i] = nt_load(reinterpret_cast<const P*>(gate) + p);
            u[i] = nt_load(reinterpret_cast<const P*>(up) + p);
        }
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            P y;
#pragma unroll
            for (int j = 0; j < VEC; ++j) y.v[j] = T::down(swiglu_fwd_1<T>(T::up(g[i].v[j]), T::up(u[i].v[j])));
            nt_store(y, reinterpret_cast<P*>(out) + p);
        }
    }
    // the last (num_elements % VEC) scalars: first lanes of block 0
    if (VEC > 1 && blockIdx.x == 0) {
        const int64_t e = num_packs * VEC + threadIdx.x;
        if (e < num_elements) out[e] = T::down(swiglu_fwd_1<T>(T::up(gate[e]), T::up(up[e])));
    }
}

template <typename T, int VEC>
__global__ void swiglu_bwd_kernel(const typename T::storage_t* __restrict__ gate,
                                  const typename T::storage_t* __restrict__ up,
                                  const typename T::storage_t* __restrict__ dy,
                                  typename T::storage_t* __restrict__ dgate,
                                  typename T::storage_t* __restrict__ dup, int64_t num_elements) {
    typedef VPack<T, VEC> P;
    const int64_t num_packs = num_elements / VEC;
    const int64_t base = (int64_t)blockIdx.x * blockDim.x * kUnroll + threadIdx.x;
    P g[kUnroll], u[kUnroll], d[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            g[i] = nt_load(reinterpret_cast<const P*>(gate) + p);
            u[i] = nt_load(reinterpret_cast<const P*>(up) + p);
            d[i] = nt_load(reinterpret_cast<const P*>(dy) + p);
        }
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < num_packs) {
            P og, ou;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                float dg, du;
                swiglu_bwd_1<T>(T::up(g[i].v[j]), T::up(u[i].v[j]), T::up(d[i].v[j]), dg, du);
                og.v[j] = T::down(dg);
                ou.v[j] = T::down(du);
            }
            nt_store(og, reinterpret_cast<P*>(dgate) + p);
            nt_store(ou, reinterpret_cast<P*>(dup) + p);
        }
    }
    if (VEC > 1 && blockIdx.x == 0) {
        const int64_t e = num_packs * VEC + threadIdx.x;
        if (e < num_elements) {
            float dg, du;
            swiglu_bwd_1<T>(T::up(gate[e]), T::up(up[e]), T::up(dy[e]), dg, du);
            dgate[e] = T::down(dg);
            dup[e] = T::down(du);
        }
    }
}

// ---- unchunked form ------------------------------------------------------------------------
// Work items are packets of the output, numbered row-major; item -> (row, column packet).
template <typename T, int VEC>
__global__ void swiglu_unchunked_fwd_kernel(const typename T::storage_t* __restrict__ x,
                                            typename T::storage_t* __restrict__ out, int64_t B, int64_t h) {
    typedef VPack<T, VEC> P;
    const int64_t packs_per_row = h / VEC;
    const int64_t total = B * packs_per_row;
    const int64_t base = (int64_t)blockIdx.x * blockDim.x * kUnroll + threadIdx.x;
    P u[kUnroll], g[kUnroll];
    int64_t row[kUnroll], col[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < total) {
            row[i] = p / packs_per_row;
            col[i] = (p - row[i] * packs_per_row) * VEC;
            const typename T::storage_t* xr = x + row[i] * 2 * h + col[i];
            u[i] = nt_load(reinterpret_cast<const P*>(xr));
            g[i] = nt_load(reinterpret_cast<const P*>(xr + h));
        }
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < total) {
            P y;
#pragma unroll
            for (int j = 0; j < VEC; ++j) y.v[j] = T::down(swiglu_fwd_1<T>(T::up(g[i].v[j]), T::up(u[i].v[j])));
            nt_store(y, reinterpret_cast<P*>(out + row[i] * h + col[i]));
        }
    }
}

template <typename T, int VEC>
__global__ void swiglu_unchunked_bwd_kernel(const typename T::storage_t* __restrict__ x,
                                            const typename T::storage_t* __restrict__ dy,
                                            typename T::storage_t* __restrict__ dx, int64_t B, int64_t h) {
    typedef VPack<T, VEC> P;
    const int64_t packs_per_row = h / VEC;
    const int64_t total = B * packs_per_row;
    const int64_t base = (int64_t)blockIdx.x * blockDim.x * kUnroll + threadIdx.x;
    P u[kUnroll], g[kUnroll], d[kUnroll];
    int64_t row[kUnroll], col[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < total) {
            row[i] = p / packs_per_row;
            col[i] = (p - row[i] * packs_per_row) * VEC;
            const typename T::storage_t* xr = x + row[i] * 2 * h + col[i];
            u[i] = nt_load(reinterpret_cast<const P*>(xr));
            g[i] = nt_load(reinterpret_cast<const P*>(xr + h));
            d[i] = nt_load(reinterpret_cast<const P*>(dy + row[i] * h + col[i]));
        }
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const int64_t p = base + (int64_t)i * blockDim.x;
        if (p < total) {
            P og, ou;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                float dg, du;
                swiglu_bwd_1<T>(T::up(g[i].v[j]), T::up(u[i].v[j]), T::up(d[i].v[j]), dg, du);
                og.v[j] = T::down(dg);
                ou.v[j] = T::down(du);
            }
            typename T::storage_t* dr = dx + row[i] * 2 * h + col[i];
            nt_store(ou, reinterpret_cast<P*>(dr));
            nt_store(og, reinterpret_cast<P*>(dr + h));
        }
    }
}

}  // namespace ck

static bool valid_block(int block_size) { return block_size >= 64 && block_size <= 1024 && block_size % 64 == 0; }

// grid for `items` work items at kUnroll per lane; false when it does not fit a 1-D grid
static bool grid_for(int64_t items, int block_size, unsigned* grid) {
    const int64_t g = items <= 0 ? 1 : ck_ceil_div(items, (int64_t)block_size * ck::kUnroll);
    if (g > 0x7fffffff) return false;
    *grid = (unsigned)g;
    return true;
}

extern "C" int ck_swiglu_forward(const void* gate, const void* up, void* output, int64_t num_elements, int dtype,
                                 int block_size, void* stream) {
    if (num_elements < 0 || !valid_block(block_size)) return CK_ERR_SHAPE;
    if (num_elements == 0) return CK_OK;
    if (!gate || !up || !output) return CK_ERR_NULL;
    if (!ck_aligned_elem(gate, dtype) || !ck_aligned_elem(up, dtype) || !ck_aligned_elem(output, dtype))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = ck_aligned16(gate) && ck_aligned16(up) && ck_aligned16(output);
    unsigned grid;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        if (vec) {
            if (!grid_for(num_elements / T::kVec, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_fwd_kernel<T, T::kVec>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)gate, (const S*)up, (S*)output, num_elements);
        } else {
            if (!grid_for(num_elements, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_fwd_kernel<T, 1>), dim3(grid), dim3(block_size), 0, s, (const S*)gate,
                               (const S*)up, (S*)output, num_elements);
        }
    });
    return ck_launch_status();
}

extern "C" int ck_swiglu_backward(const void* gate, const void* up, const void* output_grad, void* gate_grad,
                                  void* up_grad, int64_t num_elements, int dtype, int block_size, void* stream) {
    if (num_elements < 0 || !valid_block(block_size)) return CK_ERR_SHAPE;
    if (num_elements == 0) return CK_OK;
    if (!gate || !up || !output_grad || !gate_grad || !up_grad) return CK_ERR_NULL;
    const void* ptrs[5] = {gate, up, output_grad, gate_grad, up_grad};
    bool vec = true;
    for (const void* p : ptrs) {
        if (!ck_aligned_elem(p, dtype)) return CK_ERR_ALIGN;
        vec = vec && ck_aligned16(p);
    }
    hipStream_t s = (hipStream_t)stream;
    unsigned grid;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        if (vec) {
            if (!grid_for(num_elements / T::kVec, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_bwd_kernel<T, T::kVec>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)gate, (const S*)up, (const S*)output_grad, (S*)gate_grad, (S*)up_grad,
                               num_elements);
        } else {
            if (!grid_for(num_elements, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_bwd_kernel<T, 1>), dim3(grid), dim3(block_size), 0, s, (const S*)gate,
                               (const S*)up, (const S*)output_grad, (S*)gate_grad, (S*)up_grad, num_elements);
        }
    });
    return ck_launch_status();
}

extern "C" int ck_swiglu_unchunked_forward(const void* x, void* output, int64_t B, int64_t H_full, int dtype,
                                           int block_size, void* stream) {
    if (B < 0 || H_full < 0 || (H_full & 1) || !valid_block(block_size)) return CK_ERR_SHAPE;
    if (B == 0 || H_full == 0) return CK_OK;
    if (!x || !output) return CK_ERR_NULL;
    if (!ck_aligned_elem(x, dtype) || !ck_aligned_elem(output, dtype)) return CK_ERR_ALIGN;
    const int64_t h = H_full / 2;
    hipStream_t s = (hipStream_t)stream;
    unsigned grid;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(x) && ck_aligned16(output) && (h % T::kVec == 0);
        if (vec) {
            if (!grid_for(B * (h / T::kVec), block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_unchunked_fwd_kernel<T, T::kVec>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)x, (S*)output, B, h);
        } else {
            if (!grid_for(B * h, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_unchunked_fwd_kernel<T, 1>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)x, (S*)output, B, h);
        }
    });
    return ck_launch_status();
}

extern "C" int ck_swiglu_unchunked_backward(const void* x, const void* output_grad, void* x_grad, int64_t B,
                                            int64_t H_full, int dtype, int block_size, void* stream) {
    if (B < 0 || H_full < 0 || (H_full & 1) || !valid_block(block_size)) return CK_ERR_SHAPE;
    if (B == 0 || H_full == 0) return CK_OK;
    if (!x || !output_grad || !x_grad) return CK_ERR_NULL;
    if (!ck_aligned_elem(x, dtype) || !ck_aligned_elem(output_grad, dtype) || !ck_aligned_elem(x_grad, dtype))
        return CK_ERR_ALIGN;
    const int64_t h = H_full / 2;
    hipStream_t s = (hipStream_t)stream;
    unsigned grid;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(x) && ck_aligned16(output_grad) && ck_aligned16(x_grad) && (h % T::kVec == 0);
        if (vec) {
            if (!grid_for(B * (h / T::kVec), block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_unchunked_bwd_kernel<T, T::kVec>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)x, (const S*)output_grad, (S*)x_grad, B, h);
        } else {
            if (!grid_for(B * h, block_size, &grid)) return CK_ERR_SHAPE;
            hipLaunchKernelGGL((ck::swiglu_unchunked_bwd_kernel<T, 1>), dim3(grid), dim3(block_size), 0, s,
                               (const S*)x, (const S*)output_grad, (S*)x_grad, B, h);
        }
    });
    return ck_launch_status();
}
