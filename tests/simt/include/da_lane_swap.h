// Stand-in for csrc/da_lane_swap.h on the CPU: the same exchange through the simulator's lane exchange.
#pragma once
#include <hip/hip_runtime.h>

static inline float half_max(float x) { return fmaxf(x, __shfl_xor(x, 32, 64)); }
