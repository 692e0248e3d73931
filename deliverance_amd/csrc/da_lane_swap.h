// The maximum of a value over the two halves of a wavefront (lane l and lane l ^ 32), in every lane.
//
// gfx950 has an instruction that swaps the upper 32 lanes of one register with the lower 32 lanes of
// another (v_permlane32_swap_b32): given the value twice, one register then holds the lower half's values
// in both halves and the other the upper half's.  It runs on the vector unit; the general lane exchange
// (ds_bpermute_b32) goes through the LDS hardware and a wait.  Written as inline assembly: the compiler's
// own form of it returned the first result twice.
#pragma once
#include <hip/hip_runtime.h>

__device__ __forceinline__ float half_max(float x) {
  float lo = x, hi = x;
  // (two idle cycles in front, as a lane-crossing read of a register that the vector unit has just written wants)
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
  return fmaxf(lo, hi);
}
