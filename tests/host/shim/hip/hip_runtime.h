// Stand-in for <hip/hip_runtime.h> in host builds of the kernel sources (tests/host/gemm_emulation.cpp and the emulated
// library of tests/host/emulated_library.py): a workgroup is emulated as one coroutine per lane; lanes run freely and meet only where the hardware makes them meet - at workgroup
// barriers and at wave-wide instructions (shuffles, ballots, matrix instructions, transposing LDS reads), where every
// lane of the wave leaves its operand, waits for the others and computes its own result from all 64.
// Nothing here is part of the product; only the test harness includes it (through -I tests/host/shim).
#pragma once

#include <ucontext.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __restrict__
#define __align__(n) __attribute__((aligned(n)))

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
inline hipError_t hipGetLastError() { return hipSuccess; }
// the one emulated device: few compute units, so that grids sized by the device stay small
constexpr int hipDeviceAttributeMultiprocessorCount = 0;
inline hipError_t hipGetDevice(int* device) {
    *device = 0;
    return hipSuccess;
}
inline hipError_t hipDeviceGetAttribute(int* value, int, int) {
    *value = 4;
    return hipSuccess;
}
template <typename Kernel>
hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* blocks, Kernel, int, size_t) {
    *blocks = 1;
    return hipSuccess;
}
#define HIP_SYMBOL(x) (x)
template <typename Symbol>
hipError_t hipGetSymbolAddress(void** address, Symbol& symbol) {
    *address = (void*)&symbol;
    return hipSuccess;
}
struct float4 {
    float x, y, z, w;
};
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }

namespace emu {
constexpr int kWave = 64;
constexpr int kMaxLanes = 1024;
constexpr size_t kStackBytes = 512 * 1024;

struct Group {
    int arrived = 0, generation = 0, members = 0;
};
struct alignas(16) Slot {
    unsigned char bytes[48];
};
struct Wave {
    Group group;
    Slot slots[2][kWave];
};
struct Lane {
    ucontext_t context;
    std::unique_ptr<char[]> stack;  // (not a vector: its pages are touched only as deep as the lane's calls go)
    bool done = true;
    const Group* waits_for = nullptr;  // the group whose next generation this lane sleeps until
    int waits_since = 0;
};

inline ucontext_t g_main;
inline Lane g_lanes[kMaxLanes];
inline Wave g_waves[kMaxLanes / kWave];
inline Group g_block;
inline int g_current = 0, g_threads = 0;
inline dim3 g_block_index, g_grid_dim, g_block_dim;
inline std::function<void()> g_body;
inline long long g_switches = 0;

inline void yield() {
    ++g_switches;
    swapcontext(&g_lanes[g_current].context, &g_main);
}
inline void sync(Group& g) {
    const int generation = g.generation;
    if (++g.arrived >= g.members) {
        g.arrived = 0;
        ++g.generation;
    } else {
        // the scheduler resumes this lane once the last member of the group has arrived
        g_lanes[g_current].waits_for = &g;
        g_lanes[g_current].waits_since = generation;
        while (g.generation == generation) yield();
        g_lanes[g_current].waits_for = nullptr;
    }
}
inline void lane_finished() {
    // a lane that leaves the kernel no longer takes part in barriers (the hardware counts live waves)
    Group* groups[2] = {&g_block, &g_waves[g_current / kWave].group};
    for (Group* g : groups) {
        --g->members;
        if (g->members > 0 && g->arrived >= g->members) {
            g->arrived = 0;
            ++g->generation;
        }
    }
}
inline void trampoline() {
    g_body();
    g_lanes[g_current].done = true;
    lane_finished();
    swapcontext(&g_lanes[g_current].context, &g_main);
}
// hook of the harness, called once per workgroup after its last lane has left the kernel
inline std::function<void()> g_after_block;

inline bool lanes_reversed() {  // read once, when the first workgroup runs
    static const bool reversed = [] {
        const char* order = std::getenv("EMU_LANE_ORDER");
        return order != nullptr && order[0] == 'r';
    }();
    return reversed;
}

inline void run_block(int threads) {
    g_threads = threads;
    g_block = Group{};
    g_block.members = threads;
    for (int w = 0; w < (threads + kWave - 1) / kWave; ++w) {
        g_waves[w].group = Group{};
        g_waves[w].group.members = std::min(kWave, threads - w * kWave);
    }
    for (int l = 0; l < threads; ++l) {
        Lane& lane = g_lanes[l];
        if (!lane.stack) lane.stack.reset(new char[kStackBytes]);
        getcontext(&lane.context);
        lane.context.uc_stack.ss_sp = lane.stack.get();
        lane.context.uc_stack.ss_size = kStackBytes;
        lane.context.uc_link = &g_main;
        makecontext(&lane.context, trampoline, 0);
        lane.done = false;
        lane.waits_for = nullptr;
    }
    // The order in which the runnable lanes get their turn is free on the hardware; a result that depends on it is a
    // race.  EMU_LANE_ORDER=reverse runs the last lane first (default: the first lane first).
    const bool reversed = lanes_reversed();
    for (bool any = true; any;) {
        any = false;
        bool progress = false;
        for (int turn = 0; turn < threads; ++turn) {
            const int l = reversed ? threads - 1 - turn : turn;
            Lane& lane = g_lanes[l];
            if (lane.done) continue;
            any = true;
            if (lane.waits_for != nullptr && lane.waits_for->generation == lane.waits_since) continue;
            progress = true;
            g_current = l;
            swapcontext(&g_main, &lane.context);
        }
        if (any && !progress) {
            std::printf("FAILED: the workgroup hangs - every live lane waits at a barrier or a wave-wide instruction that the others never reach\n");
            std::exit(1);
        }
    }
    if (g_after_block) g_after_block();
}

template <typename Body>
void launch(dim3 grid, dim3 block, Body&& body) {
    g_grid_dim = grid;
    g_block_dim = block;
    g_body = body;
    for (unsigned z = 0; z < grid.z; ++z)
        for (unsigned y = 0; y < grid.y; ++y)
            for (unsigned x = 0; x < grid.x; ++x) {
                g_block_index = dim3(x, y, z);
                run_block((int)(block.x * block.y * block.z));
            }
}

// wave-wide instruction: every lane leaves `mine` (at most 48 bytes), then computes from all 64
template <typename In, typename F>
auto wave_instruction(const In& mine, F&& compute) {
    static_assert(sizeof(In) <= sizeof(Slot), "operand too large for the exchange slots");
    Wave& wave = g_waves[g_current / kWave];
    const int parity = wave.group.generation & 1;
    std::memcpy(wave.slots[parity][g_current % kWave].bytes, &mine, sizeof(In));
    sync(wave.group);
    return compute([&wave, parity](int lane) {
        In value;
        std::memcpy(&value, wave.slots[parity][lane].bytes, sizeof(In));
        return value;
    });
}
}  // namespace emu

#define hipLaunchKernelGGL(kernel, grid, block, shared_bytes, stream, ...) \
    emu::launch((grid), (block), [=] { kernel(__VA_ARGS__); })

struct EmuThreadIdx {
    struct X {
        operator unsigned() const { return (unsigned)emu::g_current; }
    } x;
};
struct EmuBlockIdx {
    struct X {
        operator unsigned() const { return emu::g_block_index.x; }
    } x;
    struct Y {
        operator unsigned() const { return emu::g_block_index.y; }
    } y;
    struct Z {
        operator unsigned() const { return emu::g_block_index.z; }
    } z;
};
struct EmuGridDim {
    struct X {
        operator unsigned() const { return emu::g_grid_dim.x; }
    } x;
    struct Y {
        operator unsigned() const { return emu::g_grid_dim.y; }
    } y;
};
struct EmuBlockDim {
    struct X {
        operator unsigned() const { return emu::g_block_dim.x; }
    } x;
};
inline EmuThreadIdx threadIdx;
inline EmuBlockIdx blockIdx;
inline EmuGridDim gridDim;
inline EmuBlockDim blockDim;

using std::max;
using std::min;

inline int __lane_id() { return emu::g_current % emu::kWave; }
inline void __syncthreads() { emu::sync(emu::g_block); }
// barrier that also counts the lanes whose predicate holds (three meetings: cleared by all, added by all, read by all)
inline int g_emu_votes;
inline int __syncthreads_count(int predicate) {
    g_emu_votes = 0;
    emu::sync(emu::g_block);
    g_emu_votes += predicate != 0;
    emu::sync(emu::g_block);
    const int votes = g_emu_votes;
    emu::sync(emu::g_block);
    return votes;
}
inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __popc(unsigned v) { return __builtin_popcount(v); }
inline float rsqrtf(float x) { return 1.0f / std::sqrt(x); }
// one host thread runs every lane: a read-modify-write cannot be torn
template <typename T, typename V>
T atomicAdd(T* p, V v) {
    const T old = *p;
    *p = old + (T)v;
    return old;
}
template <typename T, typename V>
T atomicMax(T* p, V v) {
    const T old = *p;
    *p = std::max(old, (T)v);
    return old;
}
inline uint64_t __ballot(bool p) {
    return emu::wave_instruction((int)p, [](auto lane) {
        uint64_t m = 0;
        for (int l = 0; l < emu::kWave; ++l) m |= (uint64_t)(lane(l) & 1) << l;
        return m;
    });
}
template <typename T>
T __shfl(T v, int src, int = 64) {
    struct In {
        T v;
        int src;
    } in{v, src};
    return emu::wave_instruction(in, [src](auto lane) { return lane(src & 63).v; });
}
template <typename T>
T __shfl_xor(T v, int mask, int = 64) {
    const int me = __lane_id();
    return emu::wave_instruction(v, [me, mask](auto lane) { return lane((me ^ mask) & 63); });
}
template <typename T>
T __shfl_up(T v, int delta, int = 64) {
    const int me = __lane_id();
    return emu::wave_instruction(v, [me, delta](auto lane) { return lane(me >= delta ? me - delta : me); });
}
inline float __expf(float x) { return std::exp(x); }

// ---- gfx950 builtins the kernel sources name directly ---------------------------------------------------------------
inline void emu_nothing() {}
inline int emu_readfirstlane(int v) {
    return emu::wave_instruction(v, [](auto lane) { return lane(0); });
}
#define __builtin_amdgcn_readfirstlane(v) emu_readfirstlane(v)
#define __builtin_amdgcn_s_barrier() emu::sync(emu::g_block)
// The lanes of a wavefront run in lock-step on the hardware; here they run freely between the instructions that make
// them meet.  Where a kernel lets lanes of one wave talk through memory and relies on the lock-step, it says so with a
// wave barrier (no instruction on the GPU, an ordering for the compiler) - here the lanes of the wave do meet there.
inline void emu_wave_barrier() { emu::sync(emu::g_waves[emu::g_current / emu::kWave].group); }
#define __builtin_amdgcn_wave_barrier() emu_wave_barrier()
#define CK_WAVE_LOCKSTEP() emu_wave_barrier()
inline void __threadfence_block() {}
inline void __threadfence() {}
#define __builtin_amdgcn_sched_barrier(mask) emu_nothing()
#define __builtin_amdgcn_s_waitcnt(code) emu_nothing()
#define __builtin_amdgcn_s_setprio(level) emu_nothing()
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))

// ---- gfx950 wave-wide instructions, modelled by their lane layouts -------------------------------------------------------
// v_mfma_f32_16x16x32: lane l holds A[i = l % 16][k = 8 (l / 16) .. + 7], B[k = 8 (l / 16) .. + 7][j = l % 16] and
// D[i = 4 (l / 16) + r][j = l % 16], r = 0 .. 3
template <typename Frag, typename Acc>
inline Acc emu_mfma16(Frag a, Frag b, Acc c) {
    struct In {
        Frag a, b;
    } in{a, b};
    const int me = __lane_id();
    return emu::wave_instruction(in, [me, c](auto lane) {
        Acc d = c;
        const int j = me % 16;
        for (int r = 0; r < 4; ++r) {
            const int i = 4 * (me / 16) + r;
            float sum = 0.f;
            for (int g = 0; g < 4; ++g) {
                const In a_lane = lane(16 * g + i), b_lane = lane(16 * g + j);
                for (int e = 0; e < 8; ++e) sum += (float)a_lane.a[e] * (float)b_lane.b[e];
            }
            d[r] += sum;
        }
        return d;
    });
}
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu_mfma16(a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) emu_mfma16(a, b, c)

// v_mfma_f32_32x32x16: lane l holds A[i = l % 32][k = 8 (l / 32) .. + 7], B likewise, and
// D[i = 8 (r / 4) + 4 (l / 32) + r % 4][j = l % 32], r = 0 .. 15
template <typename Frag, typename Acc>
inline Acc emu_mfma32(Frag a, Frag b, Acc c) {
    struct In {
        Frag a, b;
    } in{a, b};
    const int me = __lane_id();
    return emu::wave_instruction(in, [me, c](auto lane) {
        Acc d = c;
        const int j = me % 32;
        for (int r = 0; r < 16; ++r) {
            const int i = 8 * (r / 4) + 4 * (me / 32) + r % 4;
            float sum = 0.f;
            for (int g = 0; g < 2; ++g) {
                const In a_lane = lane(32 * g + i), b_lane = lane(32 * g + j);
                for (int e = 0; e < 8; ++e) sum += (float)a_lane.a[e] * (float)b_lane.b[e];
            }
            d[r] += sum;
        }
        return d;
    });
}
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) emu_mfma32(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) emu_mfma32(a, b, c)

// ds_read_b64_tr_b16: inside each group of 16 lanes, lanes 4 r .. 4 r + 3 fetch the 16 elements of row r (8 bytes
// each), and lane i receives element i of rows 0 .. 3
typedef short emu_v4i16 __attribute__((ext_vector_type(4)));
template <typename Ptr>
inline emu_v4i16 emu_ds_read_tr16(Ptr p) {
    const short* mine = (const short*)p;
    const int me = __lane_id();
    return emu::wave_instruction(mine, [me](auto lane) {
        const int group = me / 16 * 16, i = me % 16;
        emu_v4i16 out;
        for (int r = 0; r < 4; ++r) out[r] = lane(group + 4 * r + i / 4)[i % 4];
        return out;
    });
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu_ds_read_tr16(p)
