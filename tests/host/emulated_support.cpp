// Entry points of the emulated library that the kernel sources do not have: what the tests ask the emulation itself.
#include <hip/hip_runtime.h>

// 1 when this copy of the library gives the lanes of a workgroup their turns last lane first (EMU_LANE_ORDER=reverse
// in the environment when its first workgroup ran, or at this call if none has run yet)
extern "C" int emu_lanes_reversed() { return emu::lanes_reversed() ? 1 : 0; }
