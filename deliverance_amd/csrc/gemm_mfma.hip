// bfloat16 matrix products on the gfx950 matrix cores, with the epilogues a block needs:
//
//   out[m, n] (+)= act( sum_k a[m, k] * w[n, k] + bias[n] )
//
// a: [M, K] bf16, w: [N, K] bf16 ("[out, in]", K contiguous), 32-bit accumulation; out is bf16,
// or 32-bit (plain store or += for the residual stream).  Two kernels:
//
//  * gemm_tile: 128x128 block tile, 4 wavefronts of 64x64 (2x2 MFMA 32x32x16), operands staged
//    through LDS with a register prefetch of the next K-slab.  For steps with many rows (prefill).
//  * gemm_skinny: for M <= 64 (decode).  One block owns 16 output columns and all rows; its
//    wavefronts (4 to 16, by K) split K, stream their part of w straight from memory into MFMA 16x16x32
//    fragments and reduce through LDS in a fixed order.  Bound by the bytes of w.
//
// In both, an output element sums over k in an order that depends on K only, never on M or on
// the row's place in the batch.
//
// MFMA fragment layout (64 lanes).  32x32x16: lane l gives row (a) / column (b) l % 32 and the
// 8 consecutive k starting at 8 * (l / 32); it receives, for r in 0..15, the element at
// row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.  16x16x32: lane l gives row / column
// l % 16 and k = 8 * (l / 16) .. +7; it receives rows 4 * (l / 16) + r, r in 0..3, column l % 16.
#include "gemm_common.h"
#include <stdlib.h>

#define BM 128
#define BN 128
#define BKT 64               // k per slab
#define LDS_LD (BKT + 8)     // padded row length in elements (144 bytes): spreads rows over banks

// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
gemm_tile_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                 Epilogue ep, int M, int N, int K, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[BN * LDS_LD];

  // Blocks that follow each other in launch order land on different XCDs (8 of them, each with
  // its own L2).  Give each XCD a contiguous run of tiles, m fastest, so that the blocks of one
  // XCD share slabs of w.
  const int nblocks = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblocks / 8, rem = nblocks % 8;
    const int xcd = pid % 8, local = pid / 8;
    pid = xcd * per + (xcd < rem ? xcd : rem) + local;
  }
  const int tm = pid % tiles_m, tn = pid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int wm = (wave % 2) * 64, wn = (wave / 2) * 64;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // each thread moves 4 chunks of 16 bytes of each operand per slab
  uint4 ra[4], rw[4];
  const uint4 zero = make_uint4(0, 0, 0, 0);
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = t + 256 * i, row = c / 8, kc = (c % 8) * 8;
      const bool kin = k0 + kc < K;
      ra[i] = (kin && m0 + row < M) ? load16(a + (size_t)(m0 + row) * lda + k0 + kc) : zero;
      rw[i] = (kin && n0 + row < N) ? load16(w + (size_t)(n0 + row) * ldw + k0 + kc) : zero;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = t + 256 * i, row = c / 8, kc = (c % 8) * 8;
      *(uint4*)&As[row * LDS_LD + kc] = ra[i];
      *(uint4*)&Ws[row * LDS_LD + kc] = rw[i];
    }
  };

  const int fr = lane % 32, fk = (lane / 32) * 8;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BKT) {
    stash();
    __syncthreads();
    if (k0 + BKT < K) fetch(k0 + BKT);
#pragma unroll
    for (int kk = 0; kk < BKT; kk += 16) {
      bf16x8_t af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = __builtin_bit_cast(bf16x8_t, *(const uint4*)&As[(wm + i * 32 + fr) * LDS_LD + kk + fk]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[j] = __builtin_bit_cast(bf16x8_t, *(const uint4*)&Ws[(wn + j * 32 + fr) * LDS_LD + kk + fk]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn + j * 32 + fr;
    if (n >= N) continue;
    const float b = ep.bias ? load_param(ep.bias, ep.bias_dtype, n) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (m < M) epilogue_store(ep, m, n, acc[i][j][r], b);
      }
  }
}

// ---------------------------------------------------------------------------------------------
// M <= 64.  Block: 16 columns of the output, all rows; wavefront v of NW takes the k-chunks
// v, v+NW, v+2NW, ... of 32 elements each, several of them in flight at a time.  NW grows with K
// (fixed by K alone), so that the chain of dependent loads stays short.
// ---------------------------------------------------------------------------------------------
#define SK_COLS 16
template <int MT, int NW, int SK_UNROLL>   // row tiles of 16, wavefronts, k-chunks in flight per wavefront
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                   Epilogue ep, int M, int N, int K) {
  __shared__ float red[NW][MT * 16][SK_COLS + 1];
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n0 = blockIdx.x * SK_COLS;
  const int fr = lane % 16, fk = (lane / 16) * 8;
  floatx4 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  const bool wrow_ok = n0 + fr < N;
  const bf16_t* wp = w + (size_t)(wrow_ok ? n0 + fr : 0) * ldw + fk;
  bool arow_ok[MT];
  const bf16_t* ap[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    arow_ok[i] = i * 16 + fr < M;
    ap[i] = a + (size_t)(arow_ok[i] ? i * 16 + fr : 0) * lda + fk;
  }
  // what the epilogue needs is asked for first, so that it has arrived when the products are done
  constexpr int EPT = (MT * 16 * SK_COLS + NW * 64 - 1) / (NW * 64);     // output elements per thread
  float e_bias[EPT], e_old[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, m = e / SK_COLS, n = n0 + e % SK_COLS;
    const bool ok = e < MT * 16 * SK_COLS && m < M && n < N;
    e_bias[j] = (ok && ep.bias) ? load_param(ep.bias, ep.bias_dtype, n) : 0.f;
    e_old[j] = (ok && ep.accumulate) ? ((const float*)ep.out)[(size_t)m * ep.ldo + n] : 0.f;
  }
  for (int k0 = wave * 32; k0 < K; k0 += NW * 32 * SK_UNROLL) {
    uint4 wv[SK_UNROLL], av[SK_UNROLL][MT];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = k0 + u * NW * 32;
      const bool kin = k + fk < K;
      const int ks = kin ? k : -fk;             // a load that is not wanted reads the row's first chunk and is dropped
      wv[u] = load16(wp + ks);
      if (!(kin && wrow_ok)) wv[u] = zero;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        av[u][i] = load16(ap[i] + ks);
        if (!(kin && arow_ok[i])) av[u][i] = zero;
      }
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int i = 0; i < MT; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[u][i]),
                                                         __builtin_bit_cast(bf16x8_t, wv[u]), acc[i], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][i * 16 + 4 * (lane / 16) + r][fr] = acc[i][r];
  lds_barrier();
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, m = e / SK_COLS, c = e % SK_COLS, n = n0 + c;
    if (e < MT * 16 * SK_COLS && m < M && n < N) {
      float v = red[0][m][c];
#pragma unroll
      for (int v2 = 1; v2 < NW; ++v2) v += red[v2][m][c];
      v = apply_act(v + e_bias[j], ep.act);
      const size_t o = (size_t)m * ep.ldo + n;
      if (ep.accumulate) ((float*)ep.out)[o] = e_old[j] + v;
      else if (ep.out_dtype == DA_BF16) ((bf16_t*)ep.out)[o] = f32_to_bf16(v);
      else ((float*)ep.out)[o] = v;
    }
  }
}

template <int NW>
static void launch_skinny(int mt, dim3 grid, hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw,
                          const Epilogue& ep, int M, int N, int K) {
  // few rows leave registers for more chunks in flight
  if (mt == 1) hipLaunchKernelGGL((gemm_skinny_kernel<1, NW, 8>), grid, dim3(NW * 64), 0, s, A, lda, W, ldw, ep, M, N, K);
  else if (mt == 2) hipLaunchKernelGGL((gemm_skinny_kernel<2, NW, 4>), grid, dim3(NW * 64), 0, s, A, lda, W, ldw, ep, M, N, K);
  else if (mt == 3) hipLaunchKernelGGL((gemm_skinny_kernel<3, NW, 2>), grid, dim3(NW * 64), 0, s, A, lda, W, ldw, ep, M, N, K);
  else hipLaunchKernelGGL((gemm_skinny_kernel<4, NW, 2>), grid, dim3(NW * 64), 0, s, A, lda, W, ldw, ep, M, N, K);
}

extern "C" int da_gemm_bf16(const void* a, int lda, const void* w, int ldw, const void* bias, int bias_dtype,
                            int act, int accumulate, void* out, int out_dtype, int ldo, int M, int N, int K,
                            void* stream) {
  DA_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  DA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0,
             "gemm_bf16: K, lda and ldw must be multiples of 8 (K=%d lda=%d ldw=%d)", K, lda, ldw);
  DA_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  DA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_bf16: leading sizes too small");
  DA_REQUIRE(!accumulate || out_dtype == DA_F32, "gemm_bf16: accumulation needs a 32-bit output");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_SILU, "gemm_bf16: unknown activation %d", act);
  if (M == 0) return 0;
  Epilogue ep{bias, bias_dtype, act, accumulate, out, out_dtype, ldo};
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  if (M <= 64) {
    dim3 grid(da_ceil_div(N, SK_COLS));
    const int mt = da_ceil_div(M, 16);
    // the number of wavefronts that split K depends on K alone, so a row's sums keep their order
    static int force_nw = -1;
    if (force_nw < 0) { const char* e = getenv("DA_SKINNY_NW"); force_nw = e ? atoi(e) : 0; }
    int nw = K >= 2048 ? 16 : (K >= 1024 ? 8 : 4);   // measured: larger blocks cost more than they hide
    if (force_nw > 0) nw = force_nw;
    if (nw == 16) launch_skinny<16>(mt, grid, s, A, lda, W, ldw, ep, M, N, K);
    else if (nw == 8) launch_skinny<8>(mt, grid, s, A, lda, W, ldw, ep, M, N, K);
    else if (nw == 4) launch_skinny<4>(mt, grid, s, A, lda, W, ldw, ep, M, N, K);
    else launch_skinny<2>(mt, grid, s, A, lda, W, ldw, ep, M, N, K);
  } else {
    const int tiles_m = da_ceil_div(M, BM), tiles_n = da_ceil_div(N, BN);
    hipLaunchKernelGGL(gemm_tile_kernel, dim3(tiles_m * tiles_n), dim3(256), 0, s, A, lda, W, ldw, ep, M, N, K,
                       tiles_m, tiles_n);
  }
  DA_CHECK_LAUNCH("gemm_bf16");
  return 0;
}
