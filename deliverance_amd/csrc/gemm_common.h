// Shared by the matrix-core products: fragment types, the epilogue, 16-byte loads.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4s_t;   // the 4x4x4 form takes its bfloat16 as shorts

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
  v = ep.out_dtype == DA_BF16 ? apply_act_bf16(v + bias, ep.act) : apply_act(v + bias, ep.act);
  const size_t o = (size_t)m * ep.ldo + n;
  if (ep.accumulate) ((float*)ep.out)[o] += v;
  else if (ep.out_dtype == DA_BF16) ((bf16_t*)ep.out)[o] = f32_to_bf16(v);
  else ((float*)ep.out)[o] = v;
}

// For a fused q|k|v projection: the k and v columns of a row also go to the row's place in the
// paged cache (keys row-major, values dimension-major; see common.h).
struct KvScatter {
  void* cache;          // null: no scatter
  const int* slot_map;  // per row: page * page_size + row in page, or -1
  int q_cols, kv_cols;  // k occupies columns [q_cols, q_cols + kv_cols), v the next kv_cols
  int Hkv, D, page;
};

// column n (>= q_cols) of a row whose place in the cache is row `row` of page `pg`
__device__ __forceinline__ void kv_scatter_bits(const KvScatter& kv, int pg, int row, int n, bf16_t bits) {
  const int c2 = n - kv.q_cols, is_v = c2 >= kv.kv_cols, cc = is_v ? c2 - kv.kv_cols : c2;
  const int h = cc / kv.D, d = cc % kv.D;
  bf16_t* cache = (bf16_t*)kv.cache;
  if (is_v) cache[cache_v_base(pg, h, kv.Hkv, kv.page, kv.D) + (long long)d * kv.page + row] = bits;
  else cache[cache_k_row(pg, h, row, kv.Hkv, kv.page, kv.D) + d] = bits;
}

__device__ __forceinline__ void kv_scatter_store(const KvScatter& kv, int slot, int n, float v) {
  kv_scatter_bits(kv, slot / kv.page, slot % kv.page, n, f32_to_bf16(v));
}

__device__ __forceinline__ uint4 load16(const bf16_t* p) { return *(const uint4*)p; }


// The tiles whose operands go from memory straight into LDS (gemm_wide.hip): what they take, which of their
// shapes pays for a product's sizes (DA_WIDE_NONE: none), and their launch.
enum { DA_WIDE_NONE = -1, DA_WIDE_256x256 = 0, DA_WIDE_256x128 = 1, DA_WIDE_128x128 = 2 };
bool da_gemm_wide_takes(int act, int accumulate, int out_dtype, int K);
extern "C" int da_gemm_wide_choice(int M, int N, int K);
void da_gemm_wide_launch(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                         const KvScatter& kv, int M, int N, int K, int shape);
