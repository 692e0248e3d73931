// Loads from global memory straight into LDS, without a stop in registers (gfx950: 16 bytes a lane).
//
// lds_dma16(g, lds_wave_base): lane l of the wavefront copies the 16 bytes at its own `g` to
// lds_wave_base + 16 * l; `lds_wave_base` must be the same for all lanes.  The copy is asynchronous: it
// counts as a vector-memory load (vmcnt), of which the compiler knows nothing, so the kernel waits with
// DA_WAIT_VMCNT(n) (until at most n vector-memory operations of the wavefront are outstanding) and keeps
// ordinary loads out of the stretch in which it counts.  The wait goes in front of the barrier after
// which other wavefronts read the bytes.
#pragma once
#include <hip/hip_runtime.h>

__device__ __forceinline__ void lds_dma16(const void* g, void* lds_wave_base) {
  const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) void*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(base) : "memory");
}

// (lgkmcnt and expcnt are left alone: all ones in their fields)
#define DA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | (n))
