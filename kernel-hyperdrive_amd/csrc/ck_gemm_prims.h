// The instructions of the grouped GEMM that the compiler must not see through, written as assembly: the direct
// global -> LDS copy, the waits on its counter, the value fences of the optimiser, and the matrix instruction with its
// accumulator pinned to the accumulation registers.  A header of its own, behind an include guard, so that a build of
// the same kernel source for the host (tests/host/gemm_emulation.cpp) can put an emulation of each in its place by
// defining the guard first.
#ifndef CK_GEMM_PRIMS_H
#define CK_GEMM_PRIMS_H

#include "ck_device.h"

// exactly n waves of the kernel per SIMD (the LDS footprint allows no more; telling the compiler keeps it from spilling
// to reach an occupancy that cannot happen)
#define CK_WAVES_PER_SIMD(n) __attribute__((amdgpu_waves_per_eu(n, n)))

namespace ck {

// position of a byte of a __shared__ object inside the workgroup's LDS
typedef uint32_t lds_addr_t;
__device__ __forceinline__ lds_addr_t lds_address(const char* p) {
    return (lds_addr_t)(uintptr_t)((__attribute__((address_space(3))) void*)p);
}

// One copy instruction: 64 lanes x 16 bytes from (wave-uniform base + 32-bit lane offset) to the 1 KB of LDS that starts
// at `la`.  Assembly, so that the compiler's wait-count bookkeeping does not see the LDS writes: the waits for them are
// placed by hand (wait_copies).  m0 carries the LDS address of the copy; nothing else in these kernels uses it.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_copy16(lds_addr_t la, uint32_t voff, uint64_t base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(la), "v"(voff), "s"(base)
                 : "memory", "m0");
}
#pragma clang diagnostic pop

// wait until at most N of the wave's copies (vector-memory instructions) are still under way
template <int N>
__device__ __forceinline__ void wait_copies();
#define CK_WAIT_COPIES(N)                                                \
    template <>                                                          \
    __device__ __forceinline__ void wait_copies<N>() {                   \
        asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory");            \
    }
CK_WAIT_COPIES(0)
CK_WAIT_COPIES(8)
CK_WAIT_COPIES(12)
CK_WAIT_COPIES(24)
#undef CK_WAIT_COPIES

// Hides how a value was computed from the optimiser, which then cannot move the arithmetic that follows out
// of the loop and keep every variant of it alive in a register of its own.
__device__ __forceinline__ int opaque(int v) {
    asm volatile("" : "+v"(v));
    return v;
}
__device__ __forceinline__ uint64_t opaque_s64(uint64_t v) {  // same for a wave-uniform 64-bit value
    asm volatile("" : "+s"(v));
    return v;
}

// c += a x b (16 x 16 x 32) with the accumulator pinned to the accumulation half of the register file (a loop with 256
// accumulator registers per lane: left to itself the register allocator moves them between the halves)
__device__ __forceinline__ void mfma16_acc(bf16x8_t a, bf16x8_t b, f32x4_t& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma16_acc(f16x8_t a, f16x8_t b, f32x4_t& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// To the compiler the matrix instructions above are text: it does not count the wait states the hardware needs, and
// does not interlock, between a matrix instruction's write of its result and a vector-ALU or memory instruction that
// reads it (up to 18 for a 16-pass instruction) - and it is free to move such a read up to right behind them.  Called
// behind the last matrix instruction, for every row of accumulators, before the results are read: the accumulators
// pass through the statement, so no read of them can be scheduled ahead of it, and the first statement waits.
template <bool WAIT>
__device__ __forceinline__ void settle_matrix_results(f32x4_t (&c)[8]) {
    if (WAIT)
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(c[0]), "+a"(c[1]), "+a"(c[2]), "+a"(c[3]), "+a"(c[4]), "+a"(c[5]), "+a"(c[6]), "+a"(c[7]));
    else
        asm volatile("" : "+a"(c[0]), "+a"(c[1]), "+a"(c[2]), "+a"(c[3]), "+a"(c[4]), "+a"(c[5]), "+a"(c[6]), "+a"(c[7]));
}

}  // namespace ck

#endif  // CK_GEMM_PRIMS_H
