// The simulator's stand-in for deliverance_amd/csrc/da_lds_dma.h: the copy from global memory into LDS
// happens at once, lane by lane (a read outside the source tensor runs into a protected page like any
// other), and there is nothing to wait for.
#pragma once
#include <hip/hip_runtime.h>

static inline void lds_dma16(const void* g, void* lds_wave_base) {
  memcpy((char*)lds_wave_base + 16 * simt::lane_id(), g, 16);
}

#define DA_WAIT_VMCNT(n) ((void)0)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
