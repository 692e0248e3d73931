// Paged attention for prompt portions in bfloat16 on the matrix cores (flash-style: scores never
// leave the chip).  A portion's rows sit at positions past .. past+T-1 of their sequence; row i
// sees the keys lo_i .. past+i of the cache (earlier steps' keys and the portion's own, which were
// written just before).
//
// One workgroup per (portion, query head, 32 * W query rows); W wavefronts of 32 rows each.  Keys
// come in aligned tiles of 64 through two LDS buffers, two tiles ahead in registers: the key rows as they lie in the pages, the values as
// they lie in the pages too (dimension-major: a row of the LDS tile is one dimension, 64 keys).
// Per tile and wavefront, with MFMA 32x32x16:
//   S^T[key, row] = K . Q^T          keys are the MFMA's rows, so one lane holds ONE query row's
//                                     scores for 16 keys: row maximum and sum need one exchange
//                                     (lane ^ 32) instead of a reduction over the wavefront;
//   online softmax in 32-bit (maximum, exp, sum, rescale: the recurrence of
//   native/src/main/resources/decode_paged_attention_f32.wgsl:31-65);
//   O^T[dim, row] += V^T . P^T       P^T is already in registers in the layout of the B operand
//                                     (the matching, permuted order of keys is used for V^T).
// Formulas: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:458-502.
// A row's sums run over key tiles in ascending order starting at the aligned tile of its lo: the
// order depends on the row's position (and window) only.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define PF_BK 64           // keys per tile
#define PF_VLD (PF_BK + 8) // padded length of a value row in LDS
#define PF_BT_MAX 2048      // block-table entries a workgroup keeps in LDS (more are read from memory)

// head size / 16; wavefronts (32 query rows each) per workgroup; whether the block table's entries
// for the workgroup's keys fit its LDS copy (a table entry read from memory in front of a tile's loads
// makes them wait for it, and for every load still in flight)
template <int D16, int PF_WAVES, bool BT_LDS>
__global__ void __launch_bounds__(PF_WAVES * DA_WAVE)
attn_prefill_kernel(const bf16_t* __restrict__ q, int q_ld, const bf16_t* __restrict__ cache,
                    const int* __restrict__ block_table, int max_blocks,
                    const int* __restrict__ q_start, const int* __restrict__ seq_lens, int seq0,
                    int Hq, int Hkv, int page, float scale, int window,
                    bf16_t* __restrict__ out, int out_ld) {
  constexpr int D = D16 * 16;
  constexpr int DT = (D + 31) / 32;       // 32-dimension tiles of the output
  constexpr int KLD = D + 8;              // padded length of a key row in LDS
  constexpr int PF_BQ = PF_WAVES * 32;    // query rows per workgroup
  constexpr int THREADS = PF_WAVES * DA_WAVE;
  constexpr int K_PIECES = PF_BK * (D / 8), V_PIECES = DT * 32 * (PF_BK / 8);   // 16-byte pieces of a tile
  constexpr int NK = (K_PIECES + THREADS - 1) / THREADS, NV = (V_PIECES + THREADS - 1) / THREADS;  // per thread
  __shared__ __attribute__((aligned(16))) bf16_t Ks2[2][PF_BK * KLD];          // a tile is multiplied out of one
  __shared__ __attribute__((aligned(16))) bf16_t Vs2[2][DT * 32 * PF_VLD];     // while the next is parked in the other
  __shared__ int bts[PF_BT_MAX];

  const int s = seq0 + blockIdx.z, h = blockIdx.y;
  const int row0 = q_start[s], T = q_start[s + 1] - row0;
  // the workgroups with the most keys (the last rows) are launched first
  const int i0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * PF_BQ;
  if (i0 >= T) return;
  const int past = seq_lens[s] - T;
  const int hk = h / (Hq / Hkv);
  const int* bt = block_table + (size_t)s * max_blocks;
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int col = lane % 32, hf = lane / 32;

  // this lane's query row (as a column of Q^T) and its position
  const int qi = i0 + wave * 32 + col;
  const bool q_ok = qi < T;
  const int pq = past + qi;
  const int q_lo = (window > 0 && pq - window + 1 > 0) ? pq - window + 1 : 0;
  bf16x8_t qf[D16];
#pragma unroll
  for (int kd = 0; kd < D16; ++kd) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (q_ok) v = *(const uint4*)(q + (size_t)(row0 + qi) * q_ld + h * D + kd * 16 + hf * 8);
    qf[kd] = __builtin_bit_cast(bf16x8_t, v);
  }
  // the wavefront's rows span positions w_first .. w_last
  const int w_first = past + i0 + wave * 32;
  const int w_last_row = (i0 + wave * 32 + 31 < T - 1) ? i0 + wave * 32 + 31 : T - 1;
  const bool wave_on = i0 + wave * 32 < T;
  const int w_last = past + w_last_row;
  const int w_lo = (window > 0 && w_first - window + 1 > 0) ? w_first - window + 1 : 0;
  // the workgroup's keys
  const int b_last = past + ((i0 + PF_BQ - 1 < T - 1) ? i0 + PF_BQ - 1 : T - 1);
  const int b_lo = (window > 0 && past + i0 - window + 1 > 0) ? past + i0 - window + 1 : 0;

  floatx16 acc_o[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
  float m = -INFINITY, l = 0.f;                 // running maximum (base-2 domain) and sum of weights
  const float scale2 = scale * 1.4426950408889634f;

  // The next tile's keys and values are asked for (into registers) before the current tile is
  // multiplied, so their latency hides behind the arithmetic.  Loads are unconditional (a conditional
  // load becomes a branch that serialises them): a key outside b_lo .. b_last reads a key that
  // exists and is replaced by zero.
  // The block table's entries for this workgroup's keys are copied to LDS once: a table entry read
  // from memory in front of every tile would make the tile's loads wait for it, and that wait also
  // drains the loads still in flight for the tiles before.
  const int pg_lo = b_lo >> (31 - __builtin_clz(page)), pg_hi = b_last >> (31 - __builtin_clz(page));
  if (BT_LDS)
    for (int i = t; i <= pg_hi - pg_lo; i += THREADS) bts[i] = bt[pg_lo + i];
  __syncthreads();
  auto page_of = [&](int key_page) -> long long { return BT_LDS ? bts[key_page - pg_lo] : bt[key_page]; };
  // Two register sets: while a tile is multiplied, the loads of the next two are in flight.
  uint4 rk0[NK], rv0[NV], rk1[NK], rv1[NV];
  const int lg = 31 - __builtin_clz(page);              // page is a power of two (checked on the host)
  const long long page_elems = 2LL * Hkv * page * D;
  const bf16_t* kbase = cache + (long long)hk * page * D;
  const bf16_t* vbase = cache + (long long)(Hkv + hk) * page * D;
  // a tile whose 64 keys all lie in b_lo .. b_last: nothing to clamp, nothing to replace
  auto fetch_fast = [&](uint4* rk, uint4* rv, int kt) {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c0 = t + i * THREADS, c = c0 < K_PIECES ? c0 : 0;
      const int kr = c / (D / 8), pc = c % (D / 8), key = kt + kr;
      rk[i] = *(const uint4*)(kbase + page_of(key >> lg) * page_elems + (key & (page - 1)) * D + pc * 8);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c0 = t + i * THREADS, c = c0 < V_PIECES ? c0 : 0;
      const int d = c / (PF_BK / 8), g = c % (PF_BK / 8), key0 = kt + g * 8;
      const int ds = d < D ? d : 0;                      // rows of a padded 32-dimension tile repeat dimension 0
      rv[i] = *(const uint4*)(vbase + page_of(key0 >> lg) * page_elems + ds * page + (key0 & (page - 1)));
    }
  };
  auto fetch = [&](uint4* rk, uint4* rv, int kt) {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c0 = t + i * THREADS, c = c0 < K_PIECES ? c0 : 0;
      const int kr = c / (D / 8), pc = c % (D / 8), key = kt + kr;
      const bool ok = key >= b_lo && key <= b_last;
      const int ks = ok ? key : b_last;
      rk[i] = *(const uint4*)(kbase + page_of(ks >> lg) * page_elems + (ks & (page - 1)) * D + pc * 8);
      if (!ok) rk[i] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c0 = t + i * THREADS, c = c0 < V_PIECES ? c0 : 0;
      const int d = c / (PF_BK / 8), g = c % (PF_BK / 8), key0 = kt + g * 8;   // 8 keys of one dimension
      const bool ok = d < D && key0 + 7 >= b_lo && key0 <= b_last;
      const int ks = ok ? key0 : (b_last / 8) * 8;
      const int ds = d < D ? d : 0;
      uint4 v = *(const uint4*)(vbase + page_of(ks >> lg) * page_elems + ds * page + (ks & (page - 1)));
      if (!ok) v = make_uint4(0, 0, 0, 0);
      if (key0 < b_lo || key0 + 7 > b_last) {          // rows outside were never written for us
        uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (key0 + e < b_lo || key0 + e > b_last) u[e / 2] &= (e % 2) ? 0x0000ffffu : 0xffff0000u;
        v = make_uint4(u[0], u[1], u[2], u[3]);
      }
      rv[i] = v;
    }
  };
  auto stash = [&](const uint4* rk, const uint4* rv, int buf) {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c = t + i * THREADS, kr = c / (D / 8), pc = c % (D / 8);
      if (K_PIECES % THREADS == 0 || c < K_PIECES) *(uint4*)&Ks2[buf][kr * KLD + pc * 8] = rk[i];
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = t + i * THREADS, d = c / (PF_BK / 8), g = c % (PF_BK / 8);
      if (V_PIECES % THREADS == 0 || c < V_PIECES) *(uint4*)&Vs2[buf][d * PF_VLD + g * 8] = rv[i];
    }
  };
  const int kt0 = (b_lo / PF_BK) * PF_BK;
  fetch(rk0, rv0, kt0);
  if (kt0 + PF_BK <= b_last) fetch(rk1, rv1, kt0 + PF_BK);

  // the products of one tile, out of LDS buffer `buf`
  auto tile = [&](int kt, int buf) {
    const bf16_t* Ks = Ks2[buf];
    const bf16_t* Vs = Vs2[buf];
    if (wave_on && kt <= w_last && kt + PF_BK - 1 >= w_lo) {
      floatx16 sc[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[ks][r] = 0.f;
#pragma unroll
        for (int kd = 0; kd < D16; ++kd) {
          const bf16x8_t kf = __builtin_bit_cast(bf16x8_t, *(const uint4*)&Ks[(ks * 32 + col) * KLD + kd * 16 + hf * 8]);
          sc[ks] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kd], sc[ks], 0, 0, 0);
        }
      }
      // Mask, running maximum and weights.  The maximum is kept in the base-2 domain
      // (s * scale * log2 e, scale > 0), so that a weight costs one multiply-add and one hardware
      // exp2.  A tile that every row of the wavefront sees whole needs no mask at all; elsewhere a key
      // outside q_lo .. pq gets -inf added (0 otherwise), computed from the sign of
      // min(pq - key, key - q_lo) without a comparison: scores are finite, keys that do not exist
      // were loaded as zeros.
      const bool whole = kt + PF_BK - 1 <= w_first && (window <= 0 || kt >= w_last - window + 1);
      float tmax = -INFINITY;
      if (whole) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sc[ks][r]);
      } else {
        const int d0 = (q_ok ? pq : -(1 << 30)) - kt - 4 * hf;      // pq - key for the lane's first key
        const int e0 = (pq - q_lo) - d0;                             // key - q_lo likewise
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c = ks * 32 + 8 * (r / 4) + (r % 4);
            const int lo = min(d0 - c, e0 + c);
            const float bias = __builtin_bit_cast(float, (lo >> 31) & (int)0xff800000);
            const float v = sc[ks][r] + bias;
            sc[ks][r] = v;
            tmax = fmaxf(tmax, v);
          }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, DA_WAVE)) * scale2;
      const float m_new = fmaxf(m, tmax);
      const bool any = m_new != -INFINITY;             // a row that has seen no key yet keeps zeros
      const float m_use = any ? m_new : 0.f;           // -inf - 0 stays -inf: weight 0, never NaN
      const float alpha = __builtin_amdgcn_exp2f(m - m_use);
      float tsum = 0.f;
      bf16x8_t pf[2][2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          uint32_t u[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[ks][kb * 8 + 2 * e], scale2, -m_use));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[ks][kb * 8 + 2 * e + 1], scale2, -m_use));
            tsum += p0 + p1;
            u[e] = pack2_bf16(p0, p1);
          }
          pf[ks][kb] = __builtin_bit_cast(bf16x8_t, make_uint4(u[0], u[1], u[2], u[3]));
        }
      tsum += __shfl_xor(tsum, 32, DA_WAVE);
      l = l * alpha + tsum;
      m = m_new;
      // (skipping this when no row's maximum rose costs a second copy of the output's registers at
      // the branch, and with it half of the wavefronts a compute unit holds)
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] *= alpha;
      // O^T += V^T . P^T ; the lane's 8 keys of a 16-key block are 4hf..4hf+3 and 8+4hf..8+4hf+3
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
            const bf16_t* vr = &Vs[(i * 32 + col) * PF_VLD + ks * 32 + kb * 16 + 4 * hf];
            const uint2 a0 = *(const uint2*)vr, a1 = *(const uint2*)(vr + 8);
            const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, make_uint4(a0.x, a0.y, a1.x, a1.y));
            acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[ks][kb], acc_o[i], 0, 0, 0);
          }
    }
  };

  // Steady state, two tiles a round, without a branch around the loads: the compiler then counts the
  // loads in flight exactly and a tile waits for its own registers only.  It lasts while the tile
  // asked for (two ahead) lies whole inside the workgroup's keys; the last tiles run through the
  // same steps with conditions and the clamping loads.  One barrier a tile: the buffer written now
  // was last read two tiles ago, before the previous barrier.
  int kt = kt0;
  for (; kt + 4 * PF_BK - 1 <= b_last; kt += 2 * PF_BK) {
    stash(rk0, rv0, 0);
    lds_barrier();
    fetch_fast(rk0, rv0, kt + 2 * PF_BK);
    tile(kt, 0);
    stash(rk1, rv1, 1);
    lds_barrier();
    fetch_fast(rk1, rv1, kt + 3 * PF_BK);
    tile(kt + PF_BK, 1);
  }
  for (int parity = 0; kt <= b_last; kt += PF_BK, parity ^= 1) {
    if (parity == 0) {
      stash(rk0, rv0, 0);
      lds_barrier();
      if (kt + 2 * PF_BK <= b_last) fetch(rk0, rv0, kt + 2 * PF_BK);
    } else {
      stash(rk1, rv1, 1);
      lds_barrier();
      if (kt + 2 * PF_BK <= b_last) fetch(rk1, rv1, kt + 2 * PF_BK);
    }
    tile(kt, parity);
  }

  if (q_ok) {
    const float inv = 1.0f / l;
    bf16_t* orow = out + (size_t)(row0 + qi) * out_ld + h * D;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int d = i * 32 + 8 * r4 + 4 * hf;
        if (d < D) {
          const uint32_t lo2 = pack2_bf16(acc_o[i][r4 * 4] * inv, acc_o[i][r4 * 4 + 1] * inv);
          const uint32_t hi2 = pack2_bf16(acc_o[i][r4 * 4 + 2] * inv, acc_o[i][r4 * 4 + 3] * inv);
          *(uint2*)(orow + d) = make_uint2(lo2, hi2);
        }
      }
  }
}

extern "C" int da_attn_prefill(const void* q, int q_ld, const void* cache, const int* block_table,
                               int max_blocks, const int* q_start, const int* seq_lens, int seq0, int n_seqs,
                               int max_query_len, int Hq, int Hkv, int D, int page, float scale, int window,
                               void* out, int out_ld, void* stream) {
  DA_REQUIRE(n_seqs >= 0 && Hq > 0 && Hkv > 0 && page > 0 && max_query_len >= 0, "attn_prefill: bad sizes");
  DA_REQUIRE(Hq % Hkv == 0, "attn_prefill: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(D % 16 == 0 && D >= 16 && D <= 256, "attn_prefill: head size %d is not a multiple of 16 up to 256", D);
  DA_REQUIRE(page >= 8 && (page & (page - 1)) == 0 && PF_BK % page == 0, "attn_prefill: page size %d must be 8, 16, 32 or 64", page);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * D && q_ld % 8 == 0 && out_ld % 4 == 0, "attn_prefill: row lengths");
  DA_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)cache % 16 == 0) && ((uintptr_t)out % 8 == 0),
             "attn_prefill: operands must be 16-byte aligned");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_prefill: bad window or block table");
  DA_REQUIRE(scale > 0.f, "attn_prefill: the score scale must be positive, found %g", (double)scale);
  DA_REQUIRE(n_seqs <= 65535 && Hq <= 65535, "attn_prefill: too many sequences or heads for one launch");
  if (n_seqs == 0 || max_query_len == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  // every key a workgroup can see lies within max_blocks pages
  const bool bt_lds = max_blocks <= PF_BT_MAX;
#define LAUNCH2(N, W, L)                                                                                  \
  hipLaunchKernelGGL((attn_prefill_kernel<N, W, L>), dim3(da_ceil_div(max_query_len, 32 * W), Hq, n_seqs), \
                     dim3(W * DA_WAVE), 0, st, (const bf16_t*)q, q_ld, (const bf16_t*)cache, block_table, \
                     max_blocks, q_start, seq_lens, seq0, Hq, Hkv, page, scale, window, (bf16_t*)out, out_ld)
#define LAUNCH(N)                      \
  case N:                              \
    if (bt_lds) LAUNCH2(N, 4, true);   \
    else LAUNCH2(N, 4, false);         \
    break;
  switch (D / 16) {
    LAUNCH(1) LAUNCH(2) LAUNCH(3) LAUNCH(4) LAUNCH(5) LAUNCH(6) LAUNCH(7) LAUNCH(8)
    LAUNCH(9) LAUNCH(10) LAUNCH(11) LAUNCH(12) LAUNCH(13) LAUNCH(14) LAUNCH(15) LAUNCH(16)
  }
#undef LAUNCH
#undef LAUNCH2
  DA_CHECK_LAUNCH("attn_prefill");
  return 0;
}
