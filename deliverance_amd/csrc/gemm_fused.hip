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
      kv_scatter_store(kv, e_slot[j], n, apply_act_bf16(v + e_bias[j], ep.act));
  }
}

// ---------------------------------------------------------------------------------------------
// One row tile (M <= 16), K <= 2048, parameters of one dtype: every load in whole cache lines.
// Wavefront v of 8 reads rows v and v + 8 whole (RV float4 a lane), with the gain and bias at the
// same places, computes their statistics, and writes the normalised rows as bfloat16 into LDS,
// zeros past K.  The steps of w (64 elements of k, 8 rows x 128 bytes a load; wavefront v takes the
// steps v, v + 8, ...) are asked for before anything else is computed and parked in the wavefront's
// own piece of LDS; the fragments of both operands are read from LDS.  Steps past K read step 0 and
// meet zeros.  The sum over k runs in the order of the steps, whatever M is.
// TWO_ROWS false: M <= 8, a wavefront has one row and LDS holds 8 (the fragment's rows 8..15 read
// rows 0..7 again and are never stored): half the LDS, so that with a wide K two workgroups still
// share a compute unit and N / 16 workgroups run side by side.
// ---------------------------------------------------------------------------------------------
#define FL_LD (64 + 8)       // padded row of a parked step of w, elements
// CG: groups of 16 columns a workgroup (one after the other; the rows are normalised once for all of them: with a
// wide K that work, done again by every workgroup, is what the fused kernel costs, and CG workgroups' worth of it
// is saved; the next group's loads of w are asked for before this group is multiplied).
template <int RV, bool PBF16, bool TWO_ROWS, int CG = 1>
__global__ void __launch_bounds__(512)
gemm_ln_rows_kernel(LnPrologue ln, const bf16_t* __restrict__ w, int ldw, Epilogue ep, KvScatter kv,
                   int M, int N, int K) {
  constexpr int NW = 8, KMAX = RV * 256, ALD = KMAX + 8;      // ALD: padded row of a in LDS, elements
  constexpr int SW = (RV * 4 + NW - 1) / NW;                   // steps a wavefront
  constexpr int RPW = TWO_ROWS ? 2 : 1, AR = RPW * NW;         // rows a wavefront normalises; rows in LDS
  __shared__ __attribute__((aligned(16))) bf16_t a_lds[AR][ALD];
  // the wavefronts' sums take the place of the parked steps once all products are done
  constexpr int STAGE_BYTES = NW * 16 * FL_LD * 2, RED_BYTES = NW * 16 * (FZ_COLS + 1) * 4;
  __shared__ __attribute__((aligned(16))) char stage_red[STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES];
  bf16_t (*stage)[16 * FL_LD] = (bf16_t (*)[16 * FL_LD])stage_red;
  float (*red)[16][FZ_COLS + 1] = (float (*)[16][FZ_COLS + 1])stage_red;
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n_first = blockIdx.x * (FZ_COLS * CG);   // the workgroup's first column
  int n0 = n_first;                                  // the current group's first column
  const int fr = lane % 16, fk = (lane / 16) * 8;    // a fragment: row fr of 16, k-group lane / 16
  const int lr = lane / 8, lc = (lane % 8) * 8;      // a load of w: row lr of 8, 16-byte piece lane % 8

  // ---- all loads first, in the order of their use
  // (rows from M on are neither read nor normalised: what they give is never stored; the row number
  // is made a scalar so that the branch around their loads is one for the whole wavefront)
  const int row0 = __builtin_amdgcn_readfirstlane(wave);
  float4 sv[RPW][RV];
  uint4 gq[RV], bq[RV];                              // gain and bias at this lane's places (bfloat16: .x .y only)
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int m = row0 + j * NW;
    if (m < M) {
      const float* xr = ln.x + (size_t)(ln.rows ? ln.rows[m] : m) * K;
#pragma unroll
      for (int i = 0; i < RV; ++i) {
        const int c = (lane + i * 64) * 4;
        sv[j][i] = *(const float4*)(xr + (c < K ? c : 0));
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RV; ++i) {
    const int c = (lane + i * 64) * 4, cs = c < K ? c : 0;
    if (PBF16) {
      const uint2 g2 = *(const uint2*)((const bf16_t*)ln.g + cs);
      gq[i] = make_uint4(g2.x, g2.y, 0, 0);
      const uint2 b2 = *(const uint2*)((const bf16_t*)(ln.b ? ln.b : ln.g) + cs);
      bq[i] = make_uint4(b2.x, b2.y, 0, 0);
    } else {
      gq[i] = *(const uint4*)((const float*)ln.g + cs);
      bq[i] = *(const uint4*)((const float*)(ln.b ? ln.b : ln.g) + cs);
    }
  }
  // this thread's output element (16 x 16 of them) of a group, with what its epilogue needs
  const int em = t / FZ_COLS, ec = t % FZ_COLS;
  const void* e_bsrc = ep.bias ? ep.bias : (const void*)w;
  const int e_slot = kv.cache ? kv.slot_map[(t < 16 * FZ_COLS && em < M) ? em : 0] : -1;
  auto bias_bits = [&](int nfirst) -> uint32_t {
    const int en = nfirst + ec;
    const int e_bidx = (ep.bias && t < 16 * FZ_COLS && em < M && en < N) ? en : 0;
    return PBF16 ? (uint32_t)((const bf16_t*)e_bsrc)[e_bidx] : ((const uint32_t*)e_bsrc)[e_bidx];
  };
  auto ask_w = [&](uint4 (&wr)[SW][2], int nfirst) {
#pragma unroll
    for (int u = 0; u < SW; ++u) {
      const int k0 = (wave + u * NW) * 64;
      const int kk = k0 + lc < K ? k0 + lc : 0;      // past K: the row's first piece
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int n = nfirst + i * 8 + lr;
        wr[u][i] = load16(w + (size_t)(n < N ? n : 0) * ldw + kk);
      }
    }
  };
  uint32_t e_bias_raw = bias_bits(n0);
  uint4 wv[SW][2];
  ask_w(wv, n0);
  __builtin_amdgcn_sched_barrier(0);                 // the loads stay in this order, ahead of the arithmetic

  // ---- statistics and the normalised rows
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int m = row0 + j * NW;
    if (m >= M) continue;
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
#pragma unroll
    for (int i = 0; i < RV; ++i) {
      const int c = (lane + i * 64) * 4;
      float g4[4], b4[4];
      if (PBF16) {
        g4[0] = __uint_as_float(gq[i].x << 16); g4[1] = __uint_as_float(gq[i].x & 0xffff0000u);
        g4[2] = __uint_as_float(gq[i].y << 16); g4[3] = __uint_as_float(gq[i].y & 0xffff0000u);
        b4[0] = __uint_as_float(bq[i].x << 16); b4[1] = __uint_as_float(bq[i].x & 0xffff0000u);
        b4[2] = __uint_as_float(bq[i].y << 16); b4[3] = __uint_as_float(bq[i].y & 0xffff0000u);
      } else {
        g4[0] = __uint_as_float(gq[i].x); g4[1] = __uint_as_float(gq[i].y); g4[2] = __uint_as_float(gq[i].z); g4[3] = __uint_as_float(gq[i].w);
        b4[0] = __uint_as_float(bq[i].x); b4[1] = __uint_as_float(bq[i].y); b4[2] = __uint_as_float(bq[i].z); b4[3] = __uint_as_float(bq[i].w);
      }
      const float xs[4] = {sv[j][i].x, sv[j][i].y, sv[j][i].z, sv[j][i].w};
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        y[e] = (xs[e] - mean) * rstd * g4[e];
        if (ln.b) y[e] += b4[e];
      }
      uint2 pk = make_uint2((uint32_t)f32_to_bf16(y[0]) | ((uint32_t)f32_to_bf16(y[1]) << 16),
                            (uint32_t)f32_to_bf16(y[2]) | ((uint32_t)f32_to_bf16(y[3]) << 16));
      if (c >= K) pk = make_uint2(0, 0);
      *(uint2*)&a_lds[m][c] = pk;
    }
  }
  lds_barrier();

  // ---- products: a step of w is parked, then both operands' fragments come out of LDS
  bf16_t* mine = stage[wave];
#pragma unroll 1
  for (int g = 0; g < CG; ++g) {
    // the next group's w (and bias) travel while this group is multiplied
    uint4 wn[SW][2];
    uint32_t e_bias_next = 0;
    const bool more = CG > 1 && g + 1 < CG && n0 + FZ_COLS < N;
    if (CG > 1 && more) {
      ask_w(wn, n0 + FZ_COLS);
      e_bias_next = bias_bits(n0 + FZ_COLS);
    }
    floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < SW; ++u) {
      const int k0 = (wave + u * NW) * 64;             // < KMAX: the rows of a are zero from K on
#pragma unroll
      for (int i = 0; i < 2; ++i) *(uint4*)&mine[(i * 8 + lr) * FL_LD + lc] = wv[u][i];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
      if (SW * NW * 64 <= KMAX || k0 < KMAX) {
#pragma unroll
        for (int c = 0; c < 64; c += 32) {
          const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, *(const uint4*)&mine[fr * FL_LD + c + fk]);
          const bf16x8_t af = __builtin_bit_cast(bf16x8_t, *(const uint4*)&a_lds[fr % AR][k0 + c + fk]);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, wf, acc, 0, 0, 0);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
    lds_barrier();                                     // every wavefront is done with its parked steps
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * (lane / 16) + r][fr] = acc[r];
    lds_barrier();
    const int en = n0 + ec;
    if (t < 16 * FZ_COLS && em < M && en < N) {
      float v = red[0][em][ec];
#pragma unroll
      for (int v2 = 1; v2 < NW; ++v2) v += red[v2][em][ec];
      const float e_bias = !ep.bias ? 0.f : (PBF16 ? __uint_as_float(e_bias_raw << 16) : __uint_as_float(e_bias_raw));
      epilogue_store(ep, em, en, v, e_bias);
      if (kv.cache && en >= kv.q_cols && e_slot >= 0) kv_scatter_store(kv, e_slot, en, apply_act_bf16(v + e_bias, ep.act));
    }
    if (CG == 1 || !more) break;
    lds_barrier();                                     // the sums are read before the next group parks over them
    n0 += FZ_COLS;
    e_bias_raw = e_bias_next;
#pragma unroll
    for (int u = 0; u < SW; ++u) {
      wv[u][0] = wn[u][0];
      wv[u][1] = wn[u][1];
    }
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
  // the kernel with whole-line loads takes one row tile, K up to 2048, and parameters of one dtype
  // Groups of 16 columns a workgroup.  Measured on MI355X with cold weights, K = 1,600, N = 4,800 and 6,400, against
  // the norm and the product as two kernels (9.6 to 10.2 us): one group 7.9 to 8.0 us with one row, 8.4 to 8.5 with
  // 4, 10.1 with 8; two groups 8.0 to 8.2 / 7.9 to 8.5 / 9.1 to 9.6; four groups 11.8 to 13.5 (too few workgroups
  // pull on memory).  Two from 5 rows on where K is wide.
  const int groups = (M > 4 && K > 1280) ? 2 : 1;
  const int pdt = g_dtype;
  const bool same = (!b || b_dtype == pdt) && (!bias || bias_dtype == pdt) && (pdt == DA_BF16 || pdt == DA_F32);
#define LAUNCH_LDS_P(RV, PB)                                                                                      \
  do {                                                                                                            \
    if (M <= 8 && RV >= 6 && groups == 2)                                                                    \
      hipLaunchKernelGGL((gemm_ln_rows_kernel<RV, PB, false, (RV >= 6 ? 2 : 1)>), dim3(da_ceil_div(N, FZ_COLS * 2)), dim3(512), 0, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K); \
    else if (M <= 8)                                                                                              \
      hipLaunchKernelGGL((gemm_ln_rows_kernel<RV, PB, false>), grid, dim3(512), 0, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K); \
    else                                                                                                          \
      hipLaunchKernelGGL((gemm_ln_rows_kernel<RV, PB, true>), grid, dim3(512), 0, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K); \
  } while (0)
#define LAUNCH_LDS(RV)                                                                                            \
  do {                                                                                                            \
    if (pdt == DA_BF16)                                                                                           \
      LAUNCH_LDS_P(RV, true);                                                                                     \
    else                                                                                                          \
      LAUNCH_LDS_P(RV, false);                                                                                    \
  } while (0)
  if (mt == 1 && same && K <= 2048) {
    if (K <= 256) LAUNCH_LDS(1);
    else if (K <= 512) LAUNCH_LDS(2);
    else if (K <= 768) LAUNCH_LDS(3);
    else if (K <= 1024) LAUNCH_LDS(4);
    else if (K <= 1280) LAUNCH_LDS(5);
    else if (K <= 1536) LAUNCH_LDS(6);
    else if (K <= 1792) LAUNCH_LDS(7);
    else LAUNCH_LDS(8);
  } else
    // 8 wavefronts, two chunks in flight each: 125 registers, so two workgroups share a compute unit
    // (deeper unrolling needs 168 and halves that; 16 wavefronts spill)
    launch_fused<8, 2>(mt, grid, s, ln, (const bf16_t*)w, ldw, ep, kv, M, N, K);
  DA_CHECK_LAUNCH("gemm_bf16_ln");
  return 0;
}
