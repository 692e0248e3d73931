// Plain tiled matrix product with the epilogues a block needs.  This is the whole product
// path in true 32-bit (no matrix cores, no reduced-precision mode) and the reference beside
// the MFMA kernel in bfloat16.
//
//   out[m, n] (+)= act( sum_k a[m, k] * w[n, k] + bias[n] )
//
// `w` is [N, K] with K contiguous ("[out, in]"), the layout the reference multiplies against
// (tensor/src/main/java/io/teknek/deliverance/tensor/operations/NaiveTensorOperations.java:86-91).
// Every output element sums over k in the same order, whatever M is, so a row's result does
// not depend on which other rows share the step: products are summed in ascending order within
// chunks of 128, and the chunks' sums are added in ascending order (a long sum into one 32-bit
// accumulator loses about sqrt(K) roundings; in two levels it loses sqrt(128) + sqrt(K / 128)).
#include "common.h"

#define TILE 64
#define BK 16
#define CHUNK_SLABS 8      // slabs of BK that are summed before their sum joins the total

template <typename T>
__global__ void __launch_bounds__(256)
gemm_ref_kernel(const T* __restrict__ a, int lda, const T* __restrict__ w, int ldw,
                const void* __restrict__ bias, int bias_dtype, int act, int accumulate,
                void* __restrict__ out, int out_dtype, int ldo, int M, int N, int K) {
  __shared__ float As[BK][TILE + 4];
  __shared__ float Ws[BK][TILE + 4];
  const int t = threadIdx.x;
  const int tx = t % 16, ty = t / 16;
  const int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
  const int lrow = t / 4, lk = (t % 4) * 4;
  float acc[4][4], part[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = part[i][j] = 0.f;

  int slab = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + e][lrow] = (am < M && k < K) ? to_f32(a[(size_t)am * lda + k]) : 0.f;
      Ws[lk + e][lrow] = (wn < N && k < K) ? to_f32(w[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
    }
    if (++slab == CHUNK_SLABS) {
      slab = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] += part[i][j];
          part[i][j] = 0.f;
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] += part[i][j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += load_param(bias, bias_dtype, n);
      v = apply_act(v, act);
      const size_t o = (size_t)m * ldo + n;
      if (accumulate) ((float*)out)[o] += v;
      else store_out(out, out_dtype, o, v);
    }
  }
}

extern "C" int da_gemm_ref(const void* a, int lda, const void* w, int ldw, int in_dtype,
                           const void* bias, int bias_dtype, int act, int accumulate, void* out,
                           int out_dtype, int ldo, int M, int N, int K, void* stream) {
  DA_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_ref: bad sizes M=%d N=%d K=%d", M, N, K);
  DA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_ref: leading sizes too small (lda=%d ldw=%d ldo=%d)",
             lda, ldw, ldo);
  DA_REQUIRE(!accumulate || out_dtype == DA_F32, "gemm_ref: accumulation needs a 32-bit output");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_SILU, "gemm_ref: unknown activation %d", act);
  if (M == 0) return 0;
  dim3 grid(da_ceil_div(N, TILE), da_ceil_div(M, TILE));
  if (in_dtype == DA_BF16)
    hipLaunchKernelGGL(gemm_ref_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)a, lda, (const bf16_t*)w, ldw, bias, bias_dtype, act, accumulate,
                       out, out_dtype, ldo, M, N, K);
  else
    hipLaunchKernelGGL(gemm_ref_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)a, lda, (const float*)w, ldw, bias, bias_dtype, act, accumulate,
                       out, out_dtype, ldo, M, N, K);
  DA_CHECK_LAUNCH("gemm_ref");
  return 0;
}
