// Device-side helpers shared by every gfx950 kernel in this library: storage-type traits
// (fp32 / fp16 / bf16 with fp32 compute), 16-byte vector access, wave64 reductions and scans.
// Takes the place of the reference's cute_kernels/include/{dtypes/*.h,activations.h,threads.h},
// rebuilt for 64-wide wavefronts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cute_hip.h"

#define CK_WAVE 64

namespace ck {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

// ---- storage types -------------------------------------------------------------------------
struct F32 {
    typedef float storage_t;
    static constexpr int kVec = 4;  // elements per 16-byte access
    static __device__ __forceinline__ float up(storage_t v) { return v; }
    static __device__ __forceinline__ storage_t down(float v) { return v; }
};
struct F16 {
    typedef _Float16 storage_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ float up(storage_t v) { return (float)v; }
    static __device__ __forceinline__ storage_t down(float v) { return (_Float16)v; }
};
struct BF16 {
    typedef __bf16 storage_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ float up(storage_t v) { return (float)v; }
    static __device__ __forceinline__ storage_t down(float v) { return (__bf16)v; }  // RNE
};

// A packet of VEC storage elements, naturally aligned: VEC = T::kVec makes it 16 bytes.
template <typename T, int VEC>
struct alignas(sizeof(typename T::storage_t) * VEC) VPack {
    typename T::storage_t v[VEC];
};

// Streaming (non-temporal) access for any 2/4/8/16-byte POD: data touched once, keep it from
// displacing reusable cache lines.
template <int BYTES>
struct RawOf;
template <>
struct RawOf<16> {
    typedef uint32_t type __attribute__((ext_vector_type(4)));
};
template <>
struct RawOf<8> {
    typedef uint32_t type __attribute__((ext_vector_type(2)));
};
template <>
struct RawOf<4> {
    typedef uint32_t type;
};
template <>
struct RawOf<2> {
    typedef uint16_t type;
};
template <typename P>
__device__ __forceinline__ P nt_load(const P* p) {
    typedef typename RawOf<sizeof(P)>::type R;
    R raw = __builtin_nontemporal_load(reinterpret_cast<const R*>(p));
    P out;
    __builtin_memcpy(&out, &raw, sizeof(P));
    return out;
}
template <typename P>
__device__ __forceinline__ void nt_store(const P& v, P* p) {
    typedef typename RawOf<sizeof(P)>::type R;
    R raw;
    __builtin_memcpy(&raw, &v, sizeof(P));
    __builtin_nontemporal_store(raw, reinterpret_cast<R*>(p));
}

// ---- wave64 primitives ---------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return __lane_id(); }

// Marks a point where lanes of one wavefront hand data to each other through memory and rely on the wavefront's
// lock-step execution for the order (the LDS serves a wave's accesses in program order).  No instruction and no
// constraint on the GPU; a host build that runs the lanes as separate threads of control makes them meet here.
#ifndef CK_WAVE_LOCKSTEP
#define CK_WAVE_LOCKSTEP()
#endif

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, CK_WAVE);
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, CK_WAVE);
    return v;
}
// inclusive prefix sum across the 64 lanes
__device__ __forceinline__ int wave_inclusive_scan_i(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < CK_WAVE; off <<= 1) {
        int t = __shfl_up(v, off, CK_WAVE);
        if (lane >= off) v += t;
    }
    return v;
}
__device__ __forceinline__ int wave_inclusive_max_i(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < CK_WAVE; off <<= 1) {
        int t = __shfl_up(v, off, CK_WAVE);
        if (lane >= off) v = max(v, t);
    }
    return v;
}
__device__ __forceinline__ uint64_t lanemask_lt() { return (1ull << lane_id()) - 1ull; }

// Lanes of the wave whose `digit` (low `bits` bits significant) equals this lane's, via one ballot per bit.
__device__ __forceinline__ uint64_t wave_match(uint32_t digit, int bits, bool valid) {
    uint64_t m = __ballot(valid);
    for (int b = 0; b < bits; ++b) {
        const bool bit = (digit >> b) & 1u;
        const uint64_t bal = __ballot(bit);
        m &= bit ? bal : ~bal;
    }
    return m;
}

// ---- activations ---------------------------------------------------------------------------
// Exact-ish sigmoid for fp32 storage, fast-exp version for 16-bit storage (their rounding hides it).
template <typename T>
__device__ __forceinline__ float sigmoidf_(float x);
template <>
__device__ __forceinline__ float sigmoidf_<F32>(float x) {
    // evaluate on the side where exp() cannot overflow
    const float e = expf(-fabsf(x));
    const float s = 1.0f / (1.0f + e);
    return x >= 0.f ? s : 1.0f - s;
}
// (v_rcp_f32 is good to 1 ulp of fp32, far below what a 16-bit result keeps; a correctly rounded division
// costs ten more instructions per element, which shows where the activation runs in a GEMM epilogue)
template <>
__device__ __forceinline__ float sigmoidf_<F16>(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}
template <>
__device__ __forceinline__ float sigmoidf_<BF16>(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// SwiGLU of one element, y = up * gate * sigmoid(gate), and its derivatives
// (cute_kernels/kernels/swiglu/README.md:3-13); shared by the streaming kernels and the GEMM epilogues.
template <typename T>
__device__ __forceinline__ float swiglu_fwd_1(float g, float u) {
    return u * g * sigmoidf_<T>(g);
}
template <typename T>
__device__ __forceinline__ void swiglu_bwd_1(float g, float u, float dy, float& dg, float& du) {
    const float s = sigmoidf_<T>(g);
    const float gs = g * s;
    dg = dy * u * (s + gs * (1.0f - s));
    du = dy * gs;
}

}  // namespace ck

// ---- host-side helpers for the C ABI ----------------------------------------------------------
#define CK_DISPATCH_DTYPE(dtype, ...)                   \
    switch (dtype) {                                    \
        case CK_F32: {                                  \
            typedef ck::F32 T;                          \
            __VA_ARGS__;                                \
        } break;                                        \
        case CK_F16: {                                  \
            typedef ck::F16 T;                          \
            __VA_ARGS__;                                \
        } break;                                        \
        case CK_BF16: {                                 \
            typedef ck::BF16 T;                         \
            __VA_ARGS__;                                \
        } break;                                        \
        default:                                        \
            return CK_ERR_DTYPE;                        \
    }

static inline int ck_launch_status() { return hipGetLastError() == hipSuccess ? CK_OK : CK_ERR_LAUNCH; }
static inline bool ck_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int ck_elem_size(int dtype) { return dtype == CK_F32 ? 4 : 2; }
static inline bool ck_aligned_elem(const void* p, int dtype) {
    return (reinterpret_cast<uintptr_t>(p) & (uintptr_t)(ck_elem_size(dtype) - 1)) == 0;
}
static inline int64_t ck_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
