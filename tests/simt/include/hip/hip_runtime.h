// A stand-in for the HIP runtime header that lets the engine's kernel sources compile for the
// HOST, so that the kernels' own code (addressing included) can run on the CPU under guard pages.
//
// Every GPU thread of a workgroup becomes a fiber; workgroups run one after the other.  Barriers
// and cross-lane operations (DPP moves, lane reads, shuffles, matrix-core instructions) make the
// fibers of a wavefront or workgroup wait for one another, so the kernels see the data flow they
// see on the GPU.  Global memory is ordinary host memory: an access outside a tensor that was
// allocated with sim_alloc() runs into a protected page and the fault handler names the kernel,
// the workgroup, the thread and the tensor.  This is a test tool: it shares no code with the
// product and is never loaded by it.
//
// The lane layouts of the matrix-core instructions are the ones the kernels document
// (deliverance_amd/csrc/gemm_mfma.hip, header comment).
#pragma once

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define __global__
#define __device__
#define __host__
// workgroup memory: one section, so that the scheduler can fill all of it with a pattern before every
// workgroup (what a kernel reads before anyone wrote it is then a huge index or an odd number, as
// stale LDS contents can be on the GPU, and not a zero)
#define __shared__ static __attribute__((section("simt_lds")))
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct alignas(16) float4 { float x, y, z, w; };
static inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
static inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
static inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline unsigned __umulhi(unsigned a, unsigned b) { return (unsigned)(((uint64_t)a * b) >> 32); }
static inline int min(int a, int b) { return a < b ? a : b; }
static inline int max(int a, int b) { return a > b ? a : b; }

typedef void* hipStream_t;
typedef int hipError_t;
#define hipSuccess 0
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (x)
template <class T>
static inline hipError_t hipGetSymbolAddress(void** ptr, T& symbol) { *ptr = (void*)&symbol; return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "no error"; }

namespace simt {

struct Idx { unsigned x, y, z; };
struct Fiber;
extern Fiber* g_cur;                   // the fiber (GPU thread) that is running
const Idx& thread_idx();
const Idx& block_idx();
const Idx& block_dim();
const Idx& grid_dim();
int lane_id();

void block_sync();                     // __syncthreads / s_barrier
void wave_sync();                      // every live lane of the wavefront arrives
// exchange of one 32-bit word: every lane gives `v`, then reads the word of lane `src` (or of no
// lane, src < 0: `fallback`)
uint32_t lane_exchange(uint32_t v, int src, uint32_t fallback);
// the operand fragments of a matrix-core instruction: every lane gives 16 bytes of a and of b;
// afterwards frag_a(lane) / frag_b(lane) read any lane's
void frag_publish(const void* a, const void* b, int bytes);
const void* frag_a(int lane);
const void* frag_b(int lane);

typedef void (*Body)(void*);
void launch(const char* name, dim3 grid, dim3 block, Body body, void* arg);

template <class F>
static void launch_fn(const char* name, dim3 grid, dim3 block, F f) {
  launch(name, grid, block, [](void* p) { (*(F*)p)(); }, &f);
}

int dpp_source(int lane, int ctrl);    // the lane a DPP control reads from, or -1

}  // namespace simt

#define threadIdx (simt::thread_idx())
#define blockIdx (simt::block_idx())
#define blockDim (simt::block_dim())
#define gridDim (simt::grid_dim())

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  simt::launch_fn(#kernel, (grid), (block), [=]() { (kernel)(__VA_ARGS__); })

#define __syncthreads() simt::block_sync()
#define __builtin_amdgcn_s_barrier() simt::block_sync()
#define __builtin_amdgcn_wave_barrier() simt::wave_sync()
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))

static inline int simt_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool) {
  const int lane = simt::lane_id();
  const bool enabled = ((row_mask >> (lane / 16)) & 1) && ((bank_mask >> ((lane % 16) / 4)) & 1);
  const int from = enabled ? simt::dpp_source(lane, ctrl) : -1;
  return (int)simt::lane_exchange((uint32_t)src, from, (uint32_t)old);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) simt_update_dpp((old), (src), (ctrl), (rm), (bm), (bc))
static inline int simt_readlane(int v, int lane) { return (int)simt::lane_exchange((uint32_t)v, lane, 0u); }
#define __builtin_amdgcn_readlane(v, l) simt_readlane((v), (l))
#define __builtin_amdgcn_readfirstlane(v) simt_readlane((v), 0)
static inline float __shfl_xor(float v, int mask, int) {
  return __uint_as_float(simt::lane_exchange(__float_as_uint(v), simt::lane_id() ^ mask, 0u));
}
static inline int __shfl_xor(int v, int mask, int) {
  return (int)simt::lane_exchange((uint32_t)v, simt::lane_id() ^ mask, 0u);
}

// ---- matrix-core instructions ------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 simt_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float simt_floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float simt_floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short simt_shortx4;

// The products themselves live in simt_runtime.cpp (compiled with optimisation; the kernels are
// compiled without, so that every load they spell out is executed).
namespace simt {
void mfma_32x32x16(const void* a, const void* b, float* c);
void mfma_16x16x32(const void* a, const void* b, float* c);
void mfma_4x4x4(const void* a, const void* b, float* c);
}
static inline simt_floatx16 simt_mfma_32x32x16(simt_bf16x8 a, simt_bf16x8 b, simt_floatx16 c) {
  simt::mfma_32x32x16(&a, &b, (float*)&c);
  return c;
}
static inline simt_floatx4 simt_mfma_16x16x32(simt_bf16x8 a, simt_bf16x8 b, simt_floatx4 c) {
  simt::mfma_16x16x32(&a, &b, (float*)&c);
  return c;
}
static inline simt_floatx4 simt_mfma_4x4x4(simt_shortx4 a, simt_shortx4 b, simt_floatx4 c) {
  simt::mfma_4x4x4(&a, &b, (float*)&c);
  return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) simt_mfma_32x32x16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) simt_mfma_16x16x32((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(a, b, c, x, y, z) simt_mfma_4x4x4((a), (b), (c))
