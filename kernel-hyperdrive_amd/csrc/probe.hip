// Measurement aid, not part of the reference's interface: the rate the matrix cores sustain when nothing else
// runs.  Every wave keeps four groups of MFMA operands (the register footprint of the grouped GEMM's inner loop:
// 4 x 2 accumulator tiles of 32 x 32, fragments of a 128 x 64 x 64 wave tile) in registers and issues
// v_mfma_f32_32x32x16_bf16 back to back: no LDS, no memory traffic.  With all-zero operands the chip holds its
// top clock; with random operands the power limit lowers the clock, which bounds what any bf16 GEMM on real data
// can reach on this part.  The caller times the launch with events.
#include "ck_device.h"

namespace ck {

__global__ void __launch_bounds__(512) probe_mfma_kernel(const uint32_t* __restrict__ operands, int64_t iters,
                                                          float* __restrict__ sink) {
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    union Frag {
        u32x4_t raw;
        bf16x8_t f;
    };
    bf16x8_t a[4][4], b[4][2];
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(operands);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            Frag u;
            u.raw = src[(g * 6 + i) * 512 + threadIdx.x];
            a[g][i] = u.f;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            Frag u;
            u.raw = src[(g * 6 + 4 + j) * 512 + threadIdx.x];
            b[g][j] = u.f;
        }
    }
    f32x16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[g][i], b[g][j], acc[i][j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) s += acc[i][j][0];
    if (s == 12345.678f) sink[0] = s;  // keeps the loop alive; practically never true
}

}  // namespace ck

// operands: 24 * 512 * 16 bytes of bf16 data (device); sink: one float (device).  Launches `blocks` workgroups
// of 8 waves; the work is blocks * 8 * iters * 32 MFMAs of 32768 flop each.
extern "C" int ck_probe_mfma(const void* operands, int64_t iters, int blocks, float* sink, void* stream) {
    if (!operands || !sink) return CK_ERR_NULL;
    if (iters < 0 || blocks <= 0) return CK_ERR_SHAPE;
    hipLaunchKernelGGL(ck::probe_mfma_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream,
                       (const uint32_t*)operands, iters, sink);
    return ck_launch_status();
}
