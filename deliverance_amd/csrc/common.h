// Shared helpers of the gfx950 kernels: error reporting, dtype tags, bf16 conversion and
// wave-level reductions.  Every entry point is `extern "C" int da_*(...)`: it validates its
// arguments on the host, launches on the given stream and returns 0, or returns non-zero
// after storing a message that `da_last_error()` hands out.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define DA_F32 0
#define DA_BF16 1

#define DA_ACT_NONE 0
#define DA_ACT_GELU_TANH 1
#define DA_ACT_GELU_ERF 2
#define DA_ACT_RELU 3
#define DA_ACT_SILU 4

#define DA_WAVE 64

extern "C" const char* da_last_error();
void da_set_error(const char* fmt, ...);

#define DA_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      da_set_error(__VA_ARGS__);         \
      return 1;                          \
    }                                    \
  } while (0)

#define DA_CHECK_LAUNCH(name)                                                      \
  do {                                                                             \
    hipError_t e_ = hipGetLastError();                                             \
    if (e_ != hipSuccess) {                                                        \
      da_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));          \
      return 2;                                                                    \
    }                                                                              \
  } while (0)

typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest even; NaN stays a quiet NaN (the reference's C side rounds the same
// way: native/src/main/c/simd/vector_simd.c:23-41, except that it flushes subnormals).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16, quiet = (u >> 16) | 0x0040u;
  return (bf16_t)((u & 0x7fffffffu) > 0x7f800000u ? quiet : rounded);      // a select, not a branch
}

// Two floats to two bfloat16 in one word (first in the low half), round to nearest even, by the
// hardware's packed conversion.
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) float float2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const float2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T> struct DTypeOf;
template <> struct DTypeOf<float> { static const int value = DA_F32; };
template <> struct DTypeOf<bf16_t> { static const int value = DA_BF16; };

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ void from_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void from_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// Parameter vectors (norm gains, biases, tables) keep the dtype they were stored in; the
// tag travels with the pointer.
__device__ __forceinline__ float load_param(const void* p, int dtype, size_t i) {
  return dtype == DA_BF16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

__device__ __forceinline__ void store_out(void* p, int dtype, size_t i, float v) {
  if (dtype == DA_BF16) ((bf16_t*)p)[i] = f32_to_bf16(v);
  else ((float*)p)[i] = v;
}

// Reductions over the wavefront by DPP moves fused into the additions (a lane exchange through
// __shfl_xor goes through LDS hardware and costs about twenty times as much).  Every lane must be
// active.  quad_perm [1,0,3,2] and [2,3,0,1] add the lanes of a quad, row_half_mirror the two quads
// of eight lanes, row_mirror the two halves of a row of 16; row_bcast:15 and :31 carry the rows'
// totals up to lane 63, which is then read for all.  The order of the additions is fixed.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_move(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                                               CTRL, ROWMASK, 0xF, false));
}

// the sum over groups of N consecutive lanes (N a power of two), in every lane of the group
template <int N>
__device__ __forceinline__ float group_sum(float v) {
  if (N >= 2) v += dpp_move<0xB1, 0xF>(0.f, v);
  if (N >= 4) v += dpp_move<0x4E, 0xF>(0.f, v);
  if (N >= 8) v += dpp_move<0x141, 0xF>(0.f, v);
  if (N >= 16) v += dpp_move<0x140, 0xF>(0.f, v);
  if (N >= 32) v += __shfl_xor(v, 16, DA_WAVE);
  if (N >= 64) v += __shfl_xor(v, 32, DA_WAVE);
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
  v = group_sum<16>(v);
  v += dpp_move<0x142, 0xA>(0.f, v);        // rows 1 and 3 take the total of the row before
  v += dpp_move<0x143, 0xC>(0.f, v);        // rows 2 and 3 take lane 31's: row 3 now holds all four
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), DA_WAVE - 1));
}

template <int CTRL, int ROWMASK>
__device__ __forceinline__ int dpp_move_i(int old, int v) {
  return __builtin_amdgcn_update_dpp(old, v, CTRL, ROWMASK, 0xF, false);
}
template <int CTRL, int ROWMASK>
__device__ __forceinline__ double dpp_move_d(double old, double v) {
  const long long o = __builtin_bit_cast(long long, old), x = __builtin_bit_cast(long long, v);
  const unsigned lo = (unsigned)dpp_move_i<CTRL, ROWMASK>((int)o, (int)x);
  const unsigned hi = (unsigned)dpp_move_i<CTRL, ROWMASK>((int)(o >> 32), (int)(x >> 32));
  return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)lo);
}

__device__ __forceinline__ int wave_sum_i(int v) {
  v += dpp_move_i<0xB1, 0xF>(0, v);
  v += dpp_move_i<0x4E, 0xF>(0, v);
  v += dpp_move_i<0x141, 0xF>(0, v);
  v += dpp_move_i<0x140, 0xF>(0, v);
  v += dpp_move_i<0x142, 0xA>(0, v);
  v += dpp_move_i<0x143, 0xC>(0, v);
  return __builtin_amdgcn_readlane(v, DA_WAVE - 1);
}

__device__ __forceinline__ double wave_sum_d(double v) {
  v += dpp_move_d<0xB1, 0xF>(0.0, v);
  v += dpp_move_d<0x4E, 0xF>(0.0, v);
  v += dpp_move_d<0x141, 0xF>(0.0, v);
  v += dpp_move_d<0x140, 0xF>(0.0, v);
  v += dpp_move_d<0x142, 0xA>(0.0, v);
  v += dpp_move_d<0x143, 0xC>(0.0, v);
  const long long x = __builtin_bit_cast(long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)x, DA_WAVE - 1);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(x >> 32), DA_WAVE - 1);
  return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)lo);
}

// The best (value, index) pair of the wavefront under `better(a, ai, b, bi)` (a strict order), in every lane.
template <class Better>
__device__ __forceinline__ void wave_best(float& v, int& idx, Better better) {
#define DA_BEST_STEP(CTRL, ROWMASK)                                   \
  {                                                                   \
    const float ov = dpp_move<CTRL, ROWMASK>(v, v);                   \
    const int oi = dpp_move_i<CTRL, ROWMASK>(idx, idx);               \
    if (better(ov, oi, v, idx)) { v = ov; idx = oi; }                 \
  }
  DA_BEST_STEP(0xB1, 0xF) DA_BEST_STEP(0x4E, 0xF) DA_BEST_STEP(0x141, 0xF) DA_BEST_STEP(0x140, 0xF)
  DA_BEST_STEP(0x142, 0xA) DA_BEST_STEP(0x143, 0xC)
#undef DA_BEST_STEP
  v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), DA_WAVE - 1));
  idx = __builtin_amdgcn_readlane(idx, DA_WAVE - 1);
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x4E, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x141, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x140, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x142, 0xA>(v, v));
  v = fmaxf(v, dpp_move<0x143, 0xC>(v, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), DA_WAVE - 1));
}

// A workgroup barrier that orders LDS traffic only: loads from global memory that were issued
// before it stay in flight across it (a full __syncthreads waits for them).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The activations of a feed-forward, in 32-bit
// (math/src/main/java/io/teknek/deliverance/math/ActivationFunction.java:13-21).
__device__ __forceinline__ float apply_act(float x, int act) {
  switch (act) {
    case DA_ACT_GELU_TANH: {
      const float c = 0.7978845608028654f;  // sqrt(2/pi)
      return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x)));
    }
    case DA_ACT_GELU_ERF:
      return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
    case DA_ACT_RELU:
      return fmaxf(x, 0.0f);
    case DA_ACT_SILU:
      return x / (1.0f + expf(-x));
    default:
      return x;
  }
}

// One cache slot is [n_pages][2][Hkv][page * D].  Keys of a (page, head) are page rows of D
// ("row-major"); values are D runs of `page` ("dimension-major": the value of row r, dimension d
// sits at d * page + r), which is the operand layout the matrix cores want for weights x values
// and lets a decode lane own one dimension.
__device__ __forceinline__ long long cache_k_row(long long page_id, int hk, int row, int Hkv, int page, int D) {
  return page_id * (2LL * Hkv * page * D) + ((long long)hk * page + row) * D;
}
__device__ __forceinline__ long long cache_v_base(long long page_id, int hk, int Hkv, int page, int D) {
  return page_id * (2LL * Hkv * page * D) + (long long)(Hkv + hk) * page * D;
}

// The same activations where the result is rounded to bfloat16 anyway: the tanh form of GELU as
// x * sigmoid(2u), u = sqrt(2/pi) (x + 0.044715 x^3) (the same function: tanh u = 2 sigmoid(2u) - 1), with
// the hardware's exp2 and reciprocal, a few units in the last place of 32 bits off the library's tanhf
// and a fifth of its instructions.  The 32-bit path keeps apply_act.
__device__ __forceinline__ float apply_act_bf16(float x, int act) {
  if (act == DA_ACT_GELU_TANH) {
    const float u2 = 2.0f * 0.7978845608028654f * 1.4426950408889634f * (x + 0.044715f * x * x * x);   // 2u log2(e)
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-u2));
  }
  if (act == DA_ACT_SILU) return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
  return apply_act(x, act);
}

static inline int da_ceil_div(long a, long b) { return (int)((a + b - 1) / b); }
