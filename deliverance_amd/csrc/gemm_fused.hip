// Decode-sized fused product: LayerNorm of the 32-bit residual rows, the bfloat16 product on the
// matrix cores, bias / activation, and (for a q|k|v projection) the write of the new keys and
// values into the paged cache -- one kernel where a step with a handful of rows would otherwise
// pay for three.
//
//   a[m, :]   = LayerNorm(x[rows ? rows[m] : m, :]) rounded to bf16      (32-bit statistics)
//   out[m, n] = act( sum_k a[m, k] * w[n, k] + bias[n] )
//   columns n >= kv.q_cols of a q|k|v projection are also stored to the cache row kv.slot_map[m]
//
// Every block owns 16 output columns and all M <= 16*MT rows, and computes the statistics of
// all rows itself (M * K floats from L2: cheap while M is small; the host uses the unfused
// kernels for larger steps).  Statistics as in rowwise.hip: mean, then the centred sum of
// squares, one wavefront per row, the row held in registers.
// Formulas: core/src/main/java/io/teknek/deliverance/generator/LayerNorm.java:127-150,
// CausalSelfAttention.java:266-291,315-336, MLPBlock.java:250-292.
#include "gemm_common.h"

#define FZ_COLS 16
#define FZ_VPL 8          // float4 per lane when a row is held in registers: K <= 2048

struct LnPrologue {
  const float* x;
  const int* rows;
  const void* g;
  int g_dtype;
  const void* b;
  int b_dtype;
  float eps;
};

__device__ __forceinline__ void load8_param(const void* p, int dtype, int i, float* o) {
  if (dtype == DA_BF16) {
    const uint4 u = *(const uint4*)((const bf16_t*)p + i);
    const uint32_t v[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[2 * e] = __uint_as_float(v[e] << 16);
      o[2 * e + 1] = __uint_as_float(v[e] & 0xffff0000u);
    }
  } else {
    const float4 a = *(const float4*)((const float*)p + i), c = *(const float4*)((const float*)p + i + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = c.x; o[5] = c.y; o[6] = c.z; o[7] = c.w;
  }
}

template <int MT, int NW, int FZ_UNROLL>
// (for one row tile the registers are held to 128, so that two workgroups of 8 wavefronts share a compute unit)
__global__ void __launch_bounds__(NW * 64, MT == 1 ? 4 : 1)
gemm_ln_skinny_kernel(LnPrologue ln, const bf16_t* __restrict__ w, int ldw, Epilogue ep, KvScatter kv,
                      int M, int N, int K) {
  __shared__ float red[NW][MT * 16][FZ_COLS + 1];
  __shared__ float s_mean[MT * 16], s_rstd[MT * 16];
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n0 = blockIdx.x * FZ_COLS;
  const int fr = lane % 16, fk = (lane / 16) * 8;

  // The first chunks of w and of the norm's gain and bias do not depend on the statistics: their
  // loads are issued first and fly while the rows are read and reduced.
  const uint4 zero = make_uint4(0, 0, 0, 0);
  const bool wrow_ok = n0 + fr < N;
  const bf16_t* wp = w + (size_t)(wrow_ok ? n0 + fr : 0) * ldw + fk;
  uint4 wv[FZ_UNROLL];
  float gg[FZ_UNROLL][8], bb[FZ_UNROLL][8];
  auto load_wgb = [&](int k0) {
#pragma unroll
    for (int u = 0; u < FZ_UNROLL; ++u) {
      const int k = k0 + u * NW * 32;
      const bool kin = k + fk < K;
      const int ks = kin ? k : -fk;
      wv[u] = load16(wp + ks);      // past K: the row's first chunk, met by zeros in a; past N: row 0, never stored
      load8_param(ln.g, ln.g_dtype, ks + fk, gg[u]);
      if (ln.b) load8_param(ln.b, ln.b_dtype, ks + fk, bb[u]);
    }
  };
  load_wgb(wave * 32);
  // what the epilogue needs, also early: this thread's output elements are e = t, t + THREADS, ...
  constexpr int EPT = (MT * 16 * FZ_COLS + NW * 64 - 1) / (NW * 64);
  float e_bias[EPT];
  int e_slot[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, em = e / FZ_COLS, ec = e % FZ_COLS;
    const bool ok = e < MT * 16 * FZ_COLS && em < M && n0 + ec < N;
    e_bias[j] = (ok && ep.bias) ? load_param(ep.bias, ep.bias_dtype, n0 + ec) : 0.f;
    e_slot[j] = (ok && kv.cache) ? kv.slot_map[em] : -1;
  }

  // ---- statistics of every row: wavefront v takes rows v, v + NW, ...
  for (int m = wave; m < M; m += NW) {
    const float* xr = ln.x + (size_t)(ln.rows ? ln.rows[m] : m) * K;
    float4 v[FZ_VPL];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < FZ_VPL; ++i) {
      const int c = (lane + i * 64) * 4;
      v[i] = *(const float4*)(xr + (c < K ? c : 0));          // never a conditional load, nor a value replaced
      s += (c < K ? 1.f : 0.f) * ((v[i].x + v[i].y) + (v[i].z + v[i].w));
    }
    const float mean = wave_sum(s) / (float)K;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < FZ_VPL; ++i) {
      const int c = (lane + i * 64) * 4;
      if (c < K) {
        const float d0 = v[i].x - mean, d1 = v[i].y - mean, d2 = v[i].z - mean, d3 = v[i].w - mean;
        q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)K + ln.eps);
    if (lane == 0) { s_mean[m] = mean; s_rstd[m] = rstd; }
  }
  lds_barrier();

  floatx4 acc[MT];
  float mean[MT], rstd[MT];
  bool arow_ok[MT];
  const float* xp[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int m = i * 16 + fr;
    arow_ok[i] = m < M;
    const int ms = arow_ok[i] ? m : 0;
    mean[i] = s_mean[ms]; rstd[i] = s_rstd[ms];
    xp[i] = ln.x + (size_t)(ln.rows ? ln.rows[ms] : ms) * K + fk;
  }

  for (int k0 = wave * 32; k0 < K; k0 += NW * 32 * FZ_UNROLL) {
    if (k0 != wave * 32) load_wgb(k0);
    float4 xa[FZ_UNROLL][MT][2];
#pragma unroll
    for (int u = 0; u < FZ_UNROLL; ++u) {
      const int k = k0 + u * NW * 32;
      const int ks = (k + fk < K) ? k : -fk;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        xa[u][i][0] = *(const float4*)(xp[i] + ks);
        xa[u][i][1] = *(const float4*)(xp[i] + ks + 4);
      }
    }
#pragma unroll
    for (int u = 0; u < FZ_UNROLL; ++u) {
      const int k = k0 + u * NW * 32;
      const bool kin = k + fk < K;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const float xs[8] = {xa[u][i][0].x, xa[u][i][0].y, xa[u][i][0].z, xa[u][i][0].w,
                             xa[u][i][1].x, xa[u][i][1].y, xa[u][i][1].z, xa[u][i][1].w};
        uint32_t pk[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y0 = (xs[2 * e] - mean[i]) * rstd[i] * gg[u][2 * e];
          float y1 = (xs[2 * e + 1] - mean[i]) * rstd[i] * gg[u][2 * e + 1];
          if (ln.b) { y0 += bb[u][2 * e]; y1 += bb[u][2 * e + 1]; }
          pk[e] = (uint32_t)f32_to_bf16(y0) | ((uint32_t)f32_to_bf16(y1) << 16);
        }
        uint4 av = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        if (!(kin && arow_ok[i])) av = zero;
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                         __builtin_bit_cast(bf16x8_t, wv[u]), acc[i], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][i * 16 + 4 * (lane / 16) + r][fr] = acc[i][r];
  lds_barrier();
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, em = e / FZ_COLS, ec = e % FZ_COLS, n = n0 + ec;
    if (!(e < MT * 16 * FZ_COLS && em < M && n < N)) continue;
    float v = red[0][em][ec];
#pragma unroll
    for (int v2 = 1; v2 < NW; ++v2) v += red[v2][em][ec];
    epilogue_store(ep, em, n, v, e_bias[j]);
    if (kv.cache && n >= kv.q_cols && e_slot[j] >= 0)
      kv_scatter_store(kv, e_slot[j], n, apply_act(v + e_bias[j], ep.act));
  }
}

// ---------------------------------------------------------------------------------------------
// The same for up to 16 rows and K <= CH * NW * 32, with every load asked for at the start: the
// wavefront's CH chunks of w, the matching pieces of the rows, of the gain and of the bias, and the
// rows for the statistics.  The kernel then costs one memory round trip, two reductions, the
// products and the merge of the wavefronts.  Wavefront v takes the chunks v, v + NW, ...; the sum
// over k runs in that order, whatever M is.
// ---------------------------------------------------------------------------------------------
// Parameters (gain, bias of the norm, bias of the product) are loaded as raw bits and converted
// where they are used: a conversion right after its load would wait for it, and for every load
// asked for before it.  PBF16: the three are bfloat16 (else 32-bit).
template <bool PBF16>
struct Raw8 {                       // 8 consecutive parameter values as loaded
  uint4 a, b;                       // bfloat16: a only
  __device__ __forceinline__ void load(const void* p, int i) {
    if (PBF16) a = *(const uint4*)((const bf16_t*)p + i);
    else { a = *(const uint4*)((const float*)p + i); b = *(const uint4*)((const float*)p + i + 4); }
  }
  __device__ __forceinline__ void get(float* o) const {
    if (PBF16) {
      const uint32_t v[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) { o[2 * e] = __uint_as_float(v[e] << 16); o[2 * e + 1] = __uint_as_float(v[e] & 0xffff0000u); }
    } else {
      const uint32_t v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = __uint_as_float(v[e]);
    }
  }
};

// (a decode step's products have at most about one workgroup per compute unit, so registers are not held down)
template <int NW, int CH, bool PBF16>
__global__ void __launch_bounds__(NW * 64, 2)
gemm_ln_rows_kernel(LnPrologue ln, const bf16_t* __restrict__ w, int ldw, Epilogue ep, KvScatter kv,
                    int M, int N, int K) {
  constexpr int RV = (CH * NW * 32 / 4 + 63) / 64;          // float4 per lane when a row is held in registers
  __shared__ float red[NW][16][FZ_COLS + 1];
  __shared__ float s_mean[16], s_rstd[16];
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n0 = blockIdx.x * FZ_COLS;
  const int fr = lane % 16, fk = (lane / 16) * 8;
  const bool arow_ok = fr < M;
  const int arow = arow_ok ? fr : 0;
  const float* xp = ln.x + (size_t)(ln.rows ? ln.rows[arow] : arow) * K + fk;
  const bf16_t* wp = w + (size_t)(n0 + fr < N ? n0 + fr : N - 1) * ldw + fk;    // columns past N are never stored

  // Loads come back in the order they were asked for, so they are asked for in the order of their
  // use: the rows for the statistics (wavefront v takes rows v and v + NW), the pieces of the rows,
  // of the gain and of the bias for the products, what the epilogue needs, and last the chunks of w,
  // which come from furthest away.  Nothing is computed before all are on their way.
  float4 sv[2][RV];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = wave + j * NW, ms = m < M ? m : 0;
    const float* xr = ln.x + (size_t)(ln.rows ? ln.rows[ms] : ms) * K;
#pragma unroll
    for (int i = 0; i < RV; ++i) {
      const int c = (lane + i * 64) * 4;
      sv[j][i] = *(const float4*)(xr + (c < K ? c : 0));
    }
  }
  float4 xa[CH][2];
  Raw8<PBF16> gr[CH], br[CH];
  int ks[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int k = (wave + c * NW) * 32;
    ks[c] = (k + fk < K) ? k : -fk;               // past K: the row's first piece, met by zeros in a
    xa[c][0] = *(const float4*)(xp + ks[c]);
    xa[c][1] = *(const float4*)(xp + ks[c] + 4);
    gr[c].load(ln.g, ks[c] + fk);
    if (ln.b) br[c].load(ln.b, ks[c] + fk);
  }
  // this thread's output element (16 x 16 of them), with what its epilogue needs
  const int em = t / FZ_COLS, ec = t % FZ_COLS, en = n0 + ec;
  const bool e_ok = t < 16 * FZ_COLS && em < M && en < N;
  const int ebn = e_ok ? en : 0;
  // (without a bias some valid place is read and dropped: a load inside a branch is waited for there)
  const void* e_bsrc = ep.bias ? ep.bias : (const void*)w;
  const int e_bidx = ep.bias ? ebn : 0;
  const uint32_t e_bias_raw = PBF16 ? (uint32_t)((const bf16_t*)e_bsrc)[e_bidx] : ((const uint32_t*)e_bsrc)[e_bidx];
  const int e_slot = kv.cache ? kv.slot_map[e_ok ? em : 0] : -1;
  uint4 wv[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) wv[c] = load16(wp + ks[c]);
  __builtin_amdgcn_sched_barrier(0);              // the loads stay in this order, ahead of the arithmetic

  // ---- statistics
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = wave + j * NW;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < RV; ++i) {
      const int c = (lane + i * 64) * 4;
      sum += (c < K ? 1.f : 0.f) * ((sv[j][i].x + sv[j][i].y) + (sv[j][i].z + sv[j][i].w));
    }
    const float mean = wave_sum(sum) / (float)K;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < RV; ++i) {
      const int c = (lane + i * 64) * 4;
      const float d0 = sv[j][i].x - mean, d1 = sv[j][i].y - mean, d2 = sv[j][i].z - mean, d3 = sv[j][i].w - mean;
      q += (c < K ? 1.f : 0.f) * ((d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3));
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)K + ln.eps);
    if (lane == 0 && m < M) { s_mean[m] = mean; s_rstd[m] = rstd; }
  }
  lds_barrier();
  const float mean = s_mean[arow], rstd = s_rstd[arow];

  floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const bool kin = (wave + c * NW) * 32 + fk < K;
    const float xs[8] = {xa[c][0].x, xa[c][0].y, xa[c][0].z, xa[c][0].w, xa[c][1].x, xa[c][1].y, xa[c][1].z, xa[c][1].w};
    float gg[8], bb[8];
    gr[c].get(gg);
    if (ln.b) br[c].get(bb);
    uint32_t pk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float y0 = (xs[2 * e] - mean) * rstd * gg[2 * e];
      float y1 = (xs[2 * e + 1] - mean) * rstd * gg[2 * e + 1];
      if (ln.b) { y0 += bb[2 * e]; y1 += bb[2 * e + 1]; }
      pk[e] = (uint32_t)f32_to_bf16(y0) | ((uint32_t)f32_to_bf16(y1) << 16);
    }
    uint4 av = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    if (!(kin && arow_ok)) av = make_uint4(0, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, wv[c]),
                                                  acc, 0, 0, 0);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][4 * (lane / 16) + r][fr] = acc[r];
  lds_barrier();
  if (e_ok) {
    float v = red[0][em][ec];
#pragma unroll
    for (int v2 = 1; v2 < NW; ++v2) v += red[v2][em][ec];
    const float e_bias = !ep.bias ? 0.f : (PBF16 ? __uint_as_float(e_bias_raw << 16) : __uint_as_float(e_bias_raw));
    epilogue_store(ep, em, en, v, e_bias);
    if (kv.cache && en >= kv.q_cols && e_slot >= 0) kv_scatter_store(kv, e_slot, en, apply_act(v + e_bias, ep.act));
  }
}

template <int NW, int UN>
static void launch_fused(int mt, dim3 grid, hipStream_t s, const LnPrologue& ln, const bf16_t* W, int ldw,
                         const Epilogue& ep, const KvScatter& kv, int M, int N, int K) {
  if (mt == 1) hipLaunchKernelGGL((gemm_ln_skinny_kernel<1, NW, UN>), grid, dim3(NW * 64), 0, s, ln, W, ldw, ep, kv, M, N, K);
  else hipLaunchKernelGGL((gemm_ln_skinny_kernel<2, NW, UN>), grid, dim3(NW * 64), 0, s, ln, W, ldw, ep, kv, M, N, K);
}

extern "C" int da_gemm_bf16_ln(const float* x, const int* rows, const void* g, int g_dtype, const void* b,
                               int b_dtype, float eps, const void* w, int ldw, const void* bias, int bias_dtype,
                               int act, void* out, int out_dtype, int ldo, int M, int N, int K, void* kv_cache,
                               const int* slot_map, int q_cols, int kv_cols, int Hkv, int D, int page,
                               void* stream) {
  DA_REQUIRE(M > 0 && M <= 32 && N > 0 && K > 0, "gemm_bf16_ln: takes 1..32 rows (M=%d N=%d K=%d)", M, N, K);
  DA_REQUIRE(K % 8 == 0 && K <= 256 * FZ_VPL && ldw % 8 == 0 && ldw >= K && ldo >= N,
             "gemm_bf16_ln: K must be a multiple of 8 up to %d (K=%d ldw=%d)", 256 * FZ_VPL, K, ldw);
  DA_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)g % 16 == 0) &&
             (!b || (uintptr_t)b % 16 == 0), "gemm_bf16_ln: operands must be 16-byte aligned");
  DA_REQUIRE(eps > 0.f, "gemm_bf16_ln: eps must be > 0");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_SILU, "gemm_bf16_ln: unknown activation %d", act);
  if (kv_cache) {
    DA_REQUIRE(out_dtype == DA_BF16 && q_cols >= 0 && kv_cols == Hkv * D && q_cols + 2 * kv_cols == N && page > 0,
               "gemm_bf16_ln: the q|k|v columns (%d + 2*%d) must add up to N=%d", q_cols, kv_cols, N);
  }
  LnPrologue ln{x, rows, g, g_dtype, b, b_dtype, eps};
  Epilogue ep{bias, bias_dtype, act, 0, out, out_dtype, ldo};
  KvScatter kv{kv_cache, slot_map, q_cols, kv_cols, Hkv, D, page};
  dim3 grid(da_ceil_div(N, FZ_COLS));
  const int mt = da_ceil_div(M, 16);
  hipStream_t s = (hipStream_t)stream;
  // the kernel with all loads up front takes one row tile, K up to 1024, and parameters of one dtype
  const int pdt = g_dtype;
  const bool same = (!b || b_dtype == pdt) && (!bias || bias_dtype == pdt) && (pdt == DA_BF16 || pdt == DA_F32);
#define LAUNCH_ROWS(CH)                                                                                           \
  do {                                                                                                            \
    if (pdt == DA_BF16)                                                                                           \
      hipLaunchKernelGGL((gemm_ln_rows_kernel<8, CH, true>), grid, dim3(512), 0, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K); \
    else                                                                                                          \
      hipLaunchKernelGGL((gemm_ln_rows_kernel<8, CH, false>), grid, dim3(512), 0, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K); \
  } while (0)
  if (mt == 1 && same && K <= 2 * 8 * 32) LAUNCH_ROWS(2);
  else if (mt == 1 && same && K <= 3 * 8 * 32) LAUNCH_ROWS(3);
  else if (mt == 1 && same && K <= 4 * 8 * 32) LAUNCH_ROWS(4);
#undef LAUNCH_ROWS
  else
    // 8 wavefronts, two chunks in flight each: 125 registers, so two workgroups share a compute unit
    // (deeper unrolling needs 168 and halves that; 16 wavefronts spill)
    launch_fused<8, 2>(mt, grid, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K);
  DA_CHECK_LAUNCH("gemm_bf16_ln");
  return 0;
}
