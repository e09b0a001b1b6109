// The instructions behind csrc/ck_gemm_prims.h, emulated: the direct global -> LDS copy with its counter and waits, and
// the accumulating matrix instruction.  Included before the kernel source in host builds; it takes the place of the real
// header through that header's include guard.
#pragma once
#define CK_GEMM_PRIMS_H
#define CK_GEMM_PRIMS_HOST  // (a source can tell that it is being built against these models)
#define CK_WAVES_PER_SIMD(n)

#include <hip/hip_runtime.h>

#include <string>

#include "../../../kernel-hyperdrive_amd/csrc/ck_device.h"

namespace emu {
struct Region {
    const char* begin;
    const char* end;
    std::string name;
};
inline std::vector<Region> g_regions;  // global memory the kernels may read through copies (empty: not checked)
inline bool g_late_copies = false;     // copies land only when a wait forces them to (else at once)
inline int g_lax_waits = 0;            // every wait leaves this many more copies under way than it says
struct PendingCopy {
    char* dst;
    const char* src;
};
inline std::vector<PendingCopy> g_pending[kMaxLanes];
inline std::string g_case;

[[noreturn]] inline void die(const std::string& what) {
    std::printf("FAILED (%s): %s\n", g_case.c_str(), what.c_str());
    std::exit(1);
}
inline void land(const PendingCopy& c) { std::memcpy(c.dst, c.src, 16); }
}  // namespace emu

namespace ck {
typedef uintptr_t lds_addr_t;
inline lds_addr_t lds_address(const char* p) { return (lds_addr_t)p; }
inline void lds_copy16(lds_addr_t la, uint32_t voff, uint64_t base) {
    const char* src = reinterpret_cast<const char*>(base) + voff;
    bool inside = emu::g_regions.empty();
    for (const emu::Region& r : emu::g_regions) inside = inside || (src >= r.begin && src + 16 <= r.end);
    if (!inside) {
        char text[160];
        std::snprintf(text, sizeof text, "a copy reads 16 bytes at %p, outside every operand (workgroup %u, thread %d)",
                      (const void*)src, emu::g_block_index.x, emu::g_current);
        emu::die(text);
    }
    const emu::PendingCopy copy{reinterpret_cast<char*>(la) + 16 * (emu::g_current % emu::kWave), src};
    if (emu::g_late_copies)
        emu::g_pending[emu::g_current].push_back(copy);
    else
        emu::land(copy);
}
template <int N>
inline void wait_copies() {
    auto& mine = emu::g_pending[emu::g_current];
    while ((int)mine.size() > N + (N > 0 ? emu::g_lax_waits : 0)) {
        emu::land(mine.front());
        mine.erase(mine.begin());
    }
}
inline int opaque(int v) { return v; }
inline uint64_t opaque_s64(uint64_t v) { return v; }
template <bool WAIT>
inline void settle_matrix_results(f32x4_t (&)[8]) {}
inline void mfma16_acc(bf16x8_t a, bf16x8_t b, f32x4_t& c) { c = emu_mfma16(a, b, c); }
inline void mfma16_acc(f16x8_t a, f16x8_t b, f32x4_t& c) { c = emu_mfma16(a, b, c); }
}  // namespace ck
