// Stand-in for <hip/hip_runtime.h> in host builds of the kernel sources (tests/host/gemm_emulation.cpp): a workgroup is
// emulated as one coroutine per lane; lanes run freely and meet only where the hardware makes them meet - at workgroup
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
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __restrict__

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
inline hipError_t hipGetLastError() { return hipSuccess; }

namespace emu {
constexpr int kWave = 64;
constexpr int kMaxLanes = 1024;

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
    std::vector<char> stack;
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
        if (lane.stack.empty()) lane.stack.resize(512 * 1024);
        getcontext(&lane.context);
        lane.context.uc_stack.ss_sp = lane.stack.data();
        lane.context.uc_stack.ss_size = lane.stack.size();
        lane.context.uc_link = &g_main;
        makecontext(&lane.context, trampoline, 0);
        lane.done = false;
        lane.waits_for = nullptr;
    }
    for (bool any = true; any;) {
        any = false;
        bool progress = false;
        for (int l = 0; l < threads; ++l) {
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
inline EmuThreadIdx threadIdx;
inline EmuBlockIdx blockIdx;
inline EmuGridDim gridDim;

using std::max;
using std::min;

inline int __lane_id() { return emu::g_current % emu::kWave; }
inline void __syncthreads() { emu::sync(emu::g_block); }
inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
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
#define __builtin_amdgcn_sched_barrier(mask) emu_nothing()
#define __builtin_amdgcn_s_waitcnt(code) emu_nothing()
#define __builtin_amdgcn_s_setprio(level) emu_nothing()
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
