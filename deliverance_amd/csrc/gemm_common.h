// Shared by the matrix-core products: fragment types, the epilogue, 16-byte loads.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

struct Epilogue {
  const void* bias;
  int bias_dtype;
  int act;
  int accumulate;
  void* out;
  int out_dtype;
  int ldo;
};

__device__ __forceinline__ void epilogue_store(const Epilogue& ep, int m, int n, float v, float bias) {
  v = apply_act(v + bias, ep.act);
  const size_t o = (size_t)m * ep.ldo + n;
  if (ep.accumulate) ((float*)ep.out)[o] += v;
  else if (ep.out_dtype == DA_BF16) ((bf16_t*)ep.out)[o] = f32_to_bf16(v);
  else ((float*)ep.out)[o] = v;
}

__device__ __forceinline__ uint4 load16(const bf16_t* p) { return *(const uint4*)p; }

