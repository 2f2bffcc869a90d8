// Switches of the emulation that the tests flip through the built library.
#include "emu.h"

// 1: a direct-to-LDS load lands when a wait covers it (the latest the hardware allows); 0: at once.
extern "C" void emu_set_dma_late(int on) { emu::dma_late = on != 0; }

// Bytes requested by non-temporal loads since the last call (the streaming kernels read their KV tiles,
// and the merge its partial rows, with such loads).
extern "C" unsigned long long emu_take_streamed_bytes() {
  return emu::streamed_bytes.exchange(0);
}

// Bit 0: waves of a workgroup run from the last to the first; bit 1: workgroups of a launch; bit 2: lanes of a wave.
extern "C" void emu_set_run_order(int order) { emu::run_order = order; }

// Workgroups of a launch that run at the same time, each on a host thread of its own (1: one after the other).
extern "C" void emu_set_host_threads(int n) { emu::host_threads = n < 1 ? 1 : n; }
