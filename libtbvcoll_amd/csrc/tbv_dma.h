// Copy-engine transfers through the HSA runtime the process already has loaded:
// hsa_amd_memory_async_copy with a completion signal the caller polls.  No HIP
// stream and no compute queue is involved, which is what makes this path safe
// when the caller's gated stream shares a hardware queue with everything else.
#pragma once
#include <stddef.h>

namespace tbv {

enum DmaSide { DMA_DEVICE = 0, DMA_HOST = 1 };

// Finds the HSA entry points, the GPU that owns `device_ptr` and a CPU agent, and
// makes one completion signal per lane.  Returns false (and logs nothing) when
// any of that is unavailable; dma_copy then always fails.
bool dma_init(const void* device_ptr, int lanes);
void dma_fini();
bool dma_ready();

// Blocking copy of n bytes on lane `lane`'s signal; each lane is used by one
// thread at a time; lanes are independent.  A transfer that reads host memory
// uses the runtime's host-to-device engine, which works in order: it queues
// behind every host-to-device copy the process has issued before, including ones
// that wait for a stream.  Returns 0, -1 on an engine error, -2 when `timeout_s` passed.
int dma_copy(int lane, void* dst, DmaSide dst_side, const void* src, DmaSide src_side, size_t n, double timeout_s);

}  // namespace tbv
