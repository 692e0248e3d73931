// bfloat16 matrix products on the gfx950 matrix cores, with the epilogues a block needs:
//
//   out[m, n] (+)= act( sum_k a[m, k] * w[n, k] + bias[n] )
//
// a: [M, K] bf16, w: [N, K] bf16 ("[out, in]", K contiguous), 32-bit accumulation; out is bf16,
// or 32-bit (plain store or += for the residual stream).  Three kernels:
//
//  * gemm_tile: block tiles of 64x64 to 128x128 (MFMA 32x32x16), operands staged through two LDS
//    buffers, with the next four slabs already in flight in registers.  For steps with many rows
//    (prefill).  Products whose sizes suit them go to gemm_wide.hip's tiles instead (da_gemm_wide_choice).
//  * gemm_skinny: for M <= 64 (decode).  A workgroup owns 16 output columns; its wavefronts (4 to 12)
//    split K, pull their part of a and w from memory in whole cache lines, pass it through LDS into
//    MFMA 16x16x32 fragments and add their sums through LDS in a fixed order.  Bound by the bytes of w.
//  * gemm_skinny4: for M <= 4 and up to 2,048 columns.  MFMA 4x4x4, whose operand layout lets a row
//    of w be read in whole cache lines straight into registers; 4 or 8 columns a workgroup.
//
// In each, an output element sums over k in an order that depends on K only, never on M or on
// the row's place in the batch.
//
// MFMA fragment layout (64 lanes).  32x32x16: lane l gives row (a) / column (b) l % 32 and the
// 8 consecutive k starting at 8 * (l / 32); it receives, for r in 0..15, the element at
// row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.  16x16x32: lane l gives row / column
// l % 16 and k = 8 * (l / 16) .. +7; it receives rows 4 * (l / 16) + r, r in 0..3, column l % 16.
#include "gemm_common.h"
#include <type_traits>

#define BKT 64               // k per slab
#define LDS_LD (BKT + 8)     // padded row length in elements (144 bytes): spreads rows over banks

// ---------------------------------------------------------------------------------------------
// Block tile BM x BN, WM x WN wavefronts of (BM/WM) x (BN/WN) each.  Two LDS buffers: while slab k is
// multiplied out of one, the loads of slab k+1 are in flight and are then parked in the other; one
// barrier per slab.
// ---------------------------------------------------------------------------------------------
// OUTMODE: 0 bf16 store, 1 f32 store, 2 f32 +=.  ACT and OUTMODE are compile-time so that the
// epilogue is straight-line code.
// ---------------------------------------------------------------------------------------------
// The epilogue of a block tile.  A lane holds one column and 16 scattered rows of each 32 x 32 piece,
// two or four bytes wide: stored from there, a wavefront's store covers 64 bytes a row.  Instead the
// workgroup parks the tile in LDS (bias and activation applied, rounded to the output's type) and
// stores it row by row in 16-byte pieces, a whole row of the tile side by side; what += adds to is
// loaded the same way.  All loads come first and are used in straight-line code, only stores stand
// under conditions: a load under a condition would make each store wait for the one before it.
// OUTMODE: 0 bf16 store, 1 f32 store, 2 f32 +=.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN, int OUTMODE>
constexpr int tile_out_bytes() {
  return BM * (BN + (OUTMODE == 0 ? 8 : 4)) * (OUTMODE == 0 ? 2 : 4);
}
// ... and behind it, for a fused q|k|v projection, the tile rows' places in the cache
template <int BM, int OUTMODE>
constexpr int tile_slot_bytes() { return OUTMODE == 0 ? BM * 4 : 0; }

template <int BM, int BN, int WM, int WN, int ACT, int OUTMODE>
__device__ __forceinline__ void
tile_epilogue(floatx16 (&acc)[BM / WM / 32][BN / WN / 32], const float (&bias)[BN / WN / 32], char* smem, const void* safe,
              const Epilogue& ep, const KvScatter& kv, int M, int N, int m0, int n0) {
  constexpr int THREADS = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int ES = OUTMODE == 0 ? 2 : 4, CH = 16 / ES;      // bytes an element; elements a 16-byte piece
  constexpr int LDT = BN + CH;                                 // a parked row, padded by one piece
  constexpr int CPR = BN / CH, NCHK = BM * CPR / THREADS;      // pieces a row; pieces a thread
  static_assert(BM * CPR % THREADS == 0, "the tile's pieces do not split over the threads");
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int wm = (wave % WM) * (BM / WM), wn = (wave / WM) * (BN / WN);
  const int fr = lane % 32;

#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int nl = wn + j * 32 + fr;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ml = wm + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (OUTMODE == 0) ((bf16_t*)smem)[ml * LDT + nl] = f32_to_bf16(apply_act_bf16(acc[i][j][r] + bias[j], ACT));
        else ((float*)smem)[ml * LDT + nl] = apply_act(acc[i][j][r] + bias[j], ACT);
      }
  }
  lds_barrier();

  uint4 val[NCHK];
  int mm[NCHK], nn[NCHK];
#pragma unroll
  for (int k = 0; k < NCHK; ++k) {
    const int q = t + THREADS * k, row = q / CPR, c = q % CPR;
    mm[k] = m0 + row;
    nn[k] = n0 + c * CH;
    val[k] = *(const uint4*)(smem + (size_t)(row * LDT + c * CH) * ES);
  }
  const bool wide = (uintptr_t)ep.out % 16 == 0 && ep.ldo % CH == 0;
  if (wide) {
    if (OUTMODE == 2) {
      uint4 old[NCHK];
#pragma unroll
      for (int k = 0; k < NCHK; ++k) {
        const bool whole = mm[k] < M && nn[k] + CH <= N;
        old[k] = *(const uint4*)(whole ? (const void*)((const float*)ep.out + (size_t)mm[k] * ep.ldo + nn[k]) : safe);
      }
#pragma unroll
      for (int k = 0; k < NCHK; ++k) {
        const bool whole = mm[k] < M && nn[k] + CH <= N;     // (a select: what came from the safe place is dropped)
        val[k].x = whole ? __float_as_uint(__uint_as_float(old[k].x) + __uint_as_float(val[k].x)) : val[k].x;
        val[k].y = whole ? __float_as_uint(__uint_as_float(old[k].y) + __uint_as_float(val[k].y)) : val[k].y;
        val[k].z = whole ? __float_as_uint(__uint_as_float(old[k].z) + __uint_as_float(val[k].z)) : val[k].z;
        val[k].w = whole ? __float_as_uint(__uint_as_float(old[k].w) + __uint_as_float(val[k].w)) : val[k].w;
      }
    }
#pragma unroll
    for (int k = 0; k < NCHK; ++k)
      if (mm[k] < M && nn[k] + CH <= N) *(uint4*)((char*)ep.out + ((size_t)mm[k] * ep.ldo + nn[k]) * ES) = val[k];
  }
  // pieces that N cuts, and everything where the output's rows are not 16-byte aligned: by elements
  // (for +=, a piece that N cuts still holds the bare products here: only whole pieces were added to above)
#pragma unroll
  for (int k = 0; k < NCHK; ++k) {
    if (mm[k] >= M || nn[k] >= N || (wide && nn[k] + CH <= N)) continue;
    const uint32_t words[4] = {val[k].x, val[k].y, val[k].z, val[k].w};
#pragma unroll
    for (int e = 0; e < CH; ++e) {
      if (nn[k] + e >= N) continue;
      const size_t o = (size_t)mm[k] * ep.ldo + nn[k] + e;
      if (OUTMODE == 0) ((bf16_t*)ep.out)[o] = (bf16_t)(words[e / 2] >> (16 * (e % 2)));
      else if (OUTMODE == 1) ((float*)ep.out)[o] = __uint_as_float(words[e % 4]);
      else ((float*)ep.out)[o] += __uint_as_float(words[e % 4]);
    }
  }

  // A fused q|k|v projection: the k and v columns also go to the rows' places in the paged cache.
  // Keys are rows there: a piece of 8 columns is a piece of the key's row.  Values are dimension-major
  // (dimension d of a page's rows side by side): 8 consecutive tile rows of one column are one 16-byte
  // piece where their places are 8 consecutive rows of one page from a multiple of 8 on (a prompt
  // portion mostly is), and go entry by entry otherwise.
  if (OUTMODE == 0 && kv.cache) {
    int* slots = (int*)(smem + tile_out_bytes<BM, BN, OUTMODE>());      // the tile rows' places, -1: none
    for (int i = t; i < BM; i += THREADS) slots[i] = m0 + i < M ? kv.slot_map[m0 + i] : -1;
    lds_barrier();
    // (the page size is a power of two, checked on the host: a place splits into page and row by shift and mask)
    const int lgp = 31 - __builtin_clz(kv.page), pmask = kv.page - 1;
    const bool kwide = (uintptr_t)kv.cache % 16 == 0 && kv.D % 8 == 0 && kv.q_cols % 8 == 0;
    const int v0 = kv.q_cols + kv.kv_cols;                              // the first value column
#pragma unroll
    for (int k = 0; k < NCHK; ++k) {
      const int slot = slots[mm[k] - m0];
      if (slot < 0 || nn[k] >= N || nn[k] + 8 <= kv.q_cols || nn[k] >= v0) continue;
      const int pg = slot >> lgp, prow = slot & pmask;
      if (kwide) {                              // eight dimensions of one key: one piece of its row
        const int c2 = nn[k] - kv.q_cols, h = c2 / kv.D, d = c2 % kv.D;
        *(uint4*)((bf16_t*)kv.cache + cache_k_row(pg, h, prow, kv.Hkv, kv.page, kv.D) + d) = val[k];
        continue;
      }
      const uint32_t words[4] = {val[k].x, val[k].y, val[k].z, val[k].w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (nn[k] + e >= kv.q_cols && nn[k] + e < v0)
          kv_scatter_bits(kv, pg, prow, nn[k] + e, (bf16_t)(words[e / 2] >> (16 * (e % 2))));
    }
    // Values, straight from the accumulators: a lane holds 4 consecutive rows of its column (r % 4), which are 8
    // consecutive bytes of the dimension-major page when the rows' places are 4 consecutive ones from a multiple
    // of 4 on (a prompt portion's are); the lane of the other half holds the 4 rows beside them.
    const bool vwide = (uintptr_t)kv.cache % 8 == 0 && kv.page % 4 == 0;
    const long long page_stride = 2LL * kv.Hkv * kv.page * kv.D;
    bf16_t* vb = (bf16_t*)kv.cache;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn + j * 32 + fr;
      if (n < v0 || n >= N) continue;
      const int cc = n - v0;
      const int vcol = (kv.Hkv + cc / kv.D) * kv.page * kv.D + (cc % kv.D) * kv.page;   // the column's run in a page
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int r0 = wm + i * 32 + 8 * q + 4 * (lane / 32);           // the first of the lane's 4 tile rows
          const uint4 su = *(const uint4*)&slots[r0];
          const int s4[4] = {(int)su.x, (int)su.y, (int)su.z, (int)su.w};
          uint32_t w2[2];
#pragma unroll
          for (int e = 0; e < 2; ++e)
            w2[e] = pack2_bf16(apply_act_bf16(acc[i][j][4 * q + 2 * e] + bias[j], ACT),
                               apply_act_bf16(acc[i][j][4 * q + 2 * e + 1] + bias[j], ACT));
          const bool run = vwide && s4[0] >= 0 && (s4[0] & 3) == 0 && s4[1] == s4[0] + 1 && s4[2] == s4[0] + 2 && s4[3] == s4[0] + 3;
          if (run) {
            *(uint2*)(vb + (long long)(s4[0] >> lgp) * page_stride + vcol + (s4[0] & pmask)) = make_uint2(w2[0], w2[1]);
            continue;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (s4[e] >= 0)
              vb[(long long)(s4[e] >> lgp) * page_stride + vcol + (s4[e] & pmask)] = (bf16_t)(w2[e / 2] >> (16 * (e % 2)));
        }
    }
  }
}

template <int BM, int BN, int WM, int WN, int PF_SLABS, int ACT, int OUTMODE, bool KTAIL>
__device__ __forceinline__ void
gemm_tile_body(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
               const Epilogue& ep, const KvScatter& kv, int M, int N, int K, int tiles_m, int tiles_n,
               char* smem) {
  bf16_t (*As)[BM * LDS_LD] = (bf16_t (*)[BM * LDS_LD])smem;
  bf16_t (*Ws)[BN * LDS_LD] = (bf16_t (*)[BN * LDS_LD])(smem + 2 * BM * LDS_LD * sizeof(bf16_t));
  constexpr int THREADS = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;       // MFMA tiles per wavefront
  constexpr int CA = BM * 8 / THREADS, CW = BN * 8 / THREADS; // 16-byte chunks per thread and slab
  static_assert(BM * 8 % THREADS == 0 && BN * 8 % THREADS == 0, "tile does not split over the threads");
  static_assert(PF_SLABS == 2 || PF_SLABS == 4, "two or four slabs in flight");

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
  const int wm = (wave % WM) * (BM / WM), wn = (wave / WM) * (BN / WN);

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Loads are never conditional (a conditional load becomes a branch that serialises the slab's
  // loads).  Rows past the edge of a or w read the last row instead: what they produce is never
  // stored.  Chunks past K (KTAIL: K is no multiple of the slab) read the row's first chunk and are
  // replaced by zero afterwards; that replacement makes the compiler wait for loads early, so it is
  // compiled only where it is needed.  (The row's first chunk, not this thread's chunk of slab 0:
  // with K < 64 that one lies past K too, in the next row or, for the last row, past the tensor.)  PF_SLABS slabs are in flight in registers at any time: one slab's
  // products take far less time than a load, so the distance between asking and needing is what
  // keeps the matrix cores fed.
  uint4 ra[PF_SLABS][CA], rw[PF_SLABS][CW];
  const uint4 zero = make_uint4(0, 0, 0, 0);
  const bf16_t* pa[CA];
  const bf16_t* pw[CW];
#pragma unroll
  for (int i = 0; i < CA; ++i) {
    const int c = t + THREADS * i, row = m0 + c / 8;
    pa[i] = a + (size_t)(row < M ? row : M - 1) * lda + (c % 8) * 8;
  }
#pragma unroll
  for (int i = 0; i < CW; ++i) {
    const int c = t + THREADS * i, row = n0 + c / 8;
    pw[i] = w + (size_t)(row < N ? row : N - 1) * ldw + (c % 8) * 8;
  }
  const int kc_t = (t % 8) * 8;                     // this thread's chunk offset inside a slab (THREADS % 8 == 0)
#define TILE_FETCH(stage, k0)                                   \
  {                                                             \
    const bool kin = !KTAIL || (k0) + kc_t < K;                 \
    const int ks = kin ? (k0) : -kc_t;                          \
    _Pragma("unroll") for (int i = 0; i < CA; ++i) {            \
      ra[stage][i] = load16(pa[i] + ks);                        \
      if (KTAIL && !kin) ra[stage][i] = zero;                   \
    }                                                           \
    _Pragma("unroll") for (int i = 0; i < CW; ++i) {            \
      rw[stage][i] = load16(pw[i] + ks);                        \
      if (KTAIL && !kin) rw[stage][i] = zero;                   \
    }                                                           \
  }
#define TILE_STASH(stage, buf)                                              \
  {                                                                         \
    _Pragma("unroll") for (int i = 0; i < CA; ++i) {                        \
      const int c = t + THREADS * i, row = c / 8, kc = (c % 8) * 8;         \
      *(uint4*)&As[buf][row * LDS_LD + kc] = ra[stage][i];                  \
    }                                                                       \
    _Pragma("unroll") for (int i = 0; i < CW; ++i) {                        \
      const int c = t + THREADS * i, row = c / 8, kc = (c % 8) * 8;         \
      *(uint4*)&Ws[buf][row * LDS_LD + kc] = rw[stage][i];                  \
    }                                                                       \
  }
  const int fr = lane % 32, fk = (lane / 32) * 8;
  const int nslab = (K + BKT - 1) / BKT;
  // The bias is asked for now, as raw bits from a place that always exists, and has long arrived when
  // the products are done: a load inside the epilogue's conditions would make every store after it
  // wait for the one before.
  const bool bias_bf16 = ep.bias_dtype == DA_BF16;
  uint32_t braw[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn + j * 32 + fr;
    const bool has = ep.bias && n < N;
    const void* src = has ? ep.bias : (const void*)w;
    const int idx = has ? n : 0;
    braw[j] = bias_bf16 ? (uint32_t)((const bf16_t*)src)[idx] : ((const uint32_t*)src)[idx];
  }
#pragma unroll
  for (int j = 0; j < PF_SLABS; ++j)
    if (j < nslab) TILE_FETCH(j, j * BKT);
  TILE_STASH(0, 0);
  lds_barrier();
  // One slab: stage j's registers went to LDS before the last barrier and take the slab PF_SLABS
  // further on; the products of slab sidx come out of LDS buffer j & 1 (= sidx & 1, PF_SLABS is
  // even); the next slab's registers go to the other buffer, which was last read before the
  // previous barrier.
#define TILE_STEP(j, sidx, want_fetch, want_stash)                                                              \
  {                                                                                                             \
    constexpr int buf = (j) & 1;                                                                                \
    if (want_fetch) TILE_FETCH(j, ((sidx) + PF_SLABS) * BKT);                                                   \
    _Pragma("unroll") for (int kk = 0; kk < BKT; kk += 16) {                                                    \
      bf16x8_t af[TM], bf[TN];                                                                                  \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                            \
        af[i] = __builtin_bit_cast(bf16x8_t, *(const uint4*)&As[buf][(wm + i * 32 + fr) * LDS_LD + kk + fk]);   \
      _Pragma("unroll") for (int jj = 0; jj < TN; ++jj)                                                         \
        bf[jj] = __builtin_bit_cast(bf16x8_t, *(const uint4*)&Ws[buf][(wn + jj * 32 + fr) * LDS_LD + kk + fk]); \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                            \
        _Pragma("unroll") for (int jj = 0; jj < TN; ++jj)                                                       \
          acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[jj], acc[i][jj], 0, 0, 0);             \
    }                                                                                                           \
    if (want_stash) TILE_STASH(((j) + 1) % PF_SLABS, buf ^ 1);                                                  \
    lds_barrier();                                                                                              \
  }
  // The steady state has no branches, so that the compiler counts the loads in flight exactly and
  // waits for the oldest slab only; the last slabs run through the same steps with conditions.
  int base = 0;
  for (; base + 2 * PF_SLABS <= nslab; base += PF_SLABS) {
    TILE_STEP(0, base, true, true);
    TILE_STEP(1, base + 1, true, true);
    if constexpr (PF_SLABS == 4) {
      TILE_STEP(2, base + 2, true, true);
      TILE_STEP(3, base + 3, true, true);
    }
  }
  for (; base < nslab; base += PF_SLABS) {
    if (base < nslab) TILE_STEP(0, base, base + PF_SLABS < nslab, base + 1 < nslab);
    if (base + 1 < nslab) TILE_STEP(1, base + 1, base + 1 + PF_SLABS < nslab, base + 2 < nslab);
    if constexpr (PF_SLABS == 4) {
      if (base + 2 < nslab) TILE_STEP(2, base + 2, base + 2 + PF_SLABS < nslab, base + 3 < nslab);
      if (base + 3 < nslab) TILE_STEP(3, base + 3, base + 3 + PF_SLABS < nslab, base + 4 < nslab);
    }
  }
#undef TILE_STEP
#undef TILE_FETCH
#undef TILE_STASH

  float bias[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) bias[j] = !ep.bias ? 0.f : (bias_bf16 ? __uint_as_float(braw[j] << 16) : __uint_as_float(braw[j]));
  tile_epilogue<BM, BN, WM, WN, ACT, OUTMODE>(acc, bias, smem, (const void*)w, ep, kv, M, N, m0, n0);
}

template <int BM, int BN, int WM, int WN, int PF, int ACT, int OUTMODE>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_tile_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                 Epilogue ep, KvScatter kv, int M, int N, int K, int tiles_m, int tiles_n) {
  // two buffers of a slab of a and of w; the epilogue parks the tile's results in the same memory
  constexpr int SLAB_BYTES = 2 * (BM + BN) * LDS_LD * (int)sizeof(bf16_t);
  constexpr int OUT_BYTES = tile_out_bytes<BM, BN, OUTMODE>() + tile_slot_bytes<BM, OUTMODE>();
  __shared__ __attribute__((aligned(16))) char smem[SLAB_BYTES > OUT_BYTES ? SLAB_BYTES : OUT_BYTES];      // shared by the two bodies
  if (K % BKT == 0) gemm_tile_body<BM, BN, WM, WN, PF, ACT, OUTMODE, false>(a, lda, w, ldw, ep, kv, M, N, K, tiles_m, tiles_n, smem);
  else gemm_tile_body<BM, BN, WM, WN, PF, ACT, OUTMODE, true>(a, lda, w, ldw, ep, kv, M, N, K, tiles_m, tiles_n, smem);
}

template <int BM, int BN, int WM, int WN, int PF, int ACT>
static void launch_tile_act(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                            const KvScatter& kv, int M, int N, int K) {
  const int tiles_m = da_ceil_div(M, BM), tiles_n = da_ceil_div(N, BN);
  const dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  if (ep.accumulate)
    hipLaunchKernelGGL((gemm_tile_kernel<BM, BN, WM, WN, PF, ACT, 2>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
  else if (ep.out_dtype == DA_F32)
    hipLaunchKernelGGL((gemm_tile_kernel<BM, BN, WM, WN, PF, ACT, 1>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((gemm_tile_kernel<BM, BN, WM, WN, PF, ACT, 0>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
}

template <int BM, int BN, int WM, int WN, int PF>
static void launch_tile(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                        const KvScatter& kv, int M, int N, int K) {
  switch (ep.act) {
    case DA_ACT_GELU_TANH: launch_tile_act<BM, BN, WM, WN, PF, DA_ACT_GELU_TANH>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_GELU_ERF: launch_tile_act<BM, BN, WM, WN, PF, DA_ACT_GELU_ERF>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_RELU: launch_tile_act<BM, BN, WM, WN, PF, DA_ACT_RELU>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_SILU: launch_tile_act<BM, BN, WM, WN, PF, DA_ACT_SILU>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    default: launch_tile_act<BM, BN, WM, WN, PF, DA_ACT_NONE>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
  }
}

// ---------------------------------------------------------------------------------------------
// M <= 64.  A workgroup owns 16 output columns and MT row tiles of 16 (all of them, or with few
// columns some: blockIdx.y); wavefront v of NW takes the steps v, v+NW, ... of 64 elements of k, so
// that NW chains of loads run side by side; MFMA 16x16x32; the wavefronts' sums are added through
// LDS in a fixed order.  The operands come in whole cache lines: a load takes 8 rows x 128 bytes,
// the wavefront parks a step in its own piece of LDS and reads the fragments from there.  (Loaded
// straight in fragment order, 16 rows x 64 bytes a load, they pass a compute unit's L1 at a third
// of the rate, and that rate, not the memory's, bounds a workgroup.)
// ---------------------------------------------------------------------------------------------
#define SK_LD (64 + 8)       // padded row of a step in LDS, elements (144 bytes)
// AL: loads of 8 rows that cover the workgroup's rows of a (1: up to 8 rows; else two a row tile);
// COLS: 16 output columns a workgroup, or 8 (the fragment of w then holds them twice and half of the
// result is dropped: with few columns twice the workgroups pull on memory).
template <int AL, int COLS, int NW, int UNROLL>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                   Epilogue ep, KvScatter kv, int M, int N, int K) {
  constexpr int MT = (AL + 1) / 2, WL = COLS / 8;    // row tiles of 16; loads of 8 rows that cover w's columns
  constexpr int AR = MT * 16, TR = AR + COLS;        // rows of a; rows of a step: a's, then w's
  static_assert(COLS == 8 || COLS == 16, "8 or 16 columns a workgroup");
  // the wavefronts' partial sums take the place of the parked steps once all products are done
  constexpr int STAGE_BYTES = NW * TR * SK_LD * 2, RED_BYTES = NW * AR * (COLS + 1) * 4;
  __shared__ __attribute__((aligned(16))) char smem[STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES];
  bf16_t (*stage)[TR * SK_LD] = (bf16_t (*)[TR * SK_LD])smem;
  float (*red)[AR][COLS + 1] = (float (*)[AR][COLS + 1])smem;
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n0 = blockIdx.x * COLS;
  const int r0 = blockIdx.y * AR;                    // the workgroup's first row
  const int lr = lane / 8, lc = (lane % 8) * 8;      // a load: row lr of 8, 16-byte piece lane % 8
  const int fr = lane % 16, fk = (lane / 16) * 8;    // a fragment: row fr of 16, k-group lane / 16
  const bf16_t* pa[AL];
  const bf16_t* pw[WL];
#pragma unroll
  for (int i = 0; i < AL; ++i) {
    const int m = r0 + i * 8 + lr;
    pa[i] = a + (size_t)(m < M ? m : 0) * lda + lc;
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int n = n0 + i * 8 + lr;
    pw[i] = w + (size_t)(n < N ? n : 0) * ldw + lc;
  }
  // what the epilogue needs is asked for first, as raw bits from places that always exist
  constexpr int EPT = (AR * COLS + NW * 64 - 1) / (NW * 64);
  uint32_t e_braw[EPT];
  float e_old[EPT];
  int e_slot[EPT];
  const bool bias_bf16 = ep.bias_dtype == DA_BF16;
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, m = r0 + e / COLS, n = n0 + e % COLS;
    const bool ok = e < AR * COLS && m < M && n < N;
    const void* bsrc = (ok && ep.bias) ? ep.bias : (const void*)w;
    const int bidx = (ok && ep.bias) ? n : 0;
    e_braw[j] = bias_bf16 ? (uint32_t)((const bf16_t*)bsrc)[bidx] : ((const uint32_t*)bsrc)[bidx];
    e_old[j] = *((ok && ep.accumulate) ? (const float*)ep.out + (size_t)m * ep.ldo + n : (const float*)w);
    e_slot[j] = *((ok && kv.cache) ? kv.slot_map + m : (const int*)w);
  }
  floatx4 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16_t* mine = stage[wave];
  // (With AL == 1 the rows 8..15 of the tile are never parked: whatever LDS holds there gives rows of
  // the result that are never stored.)
  // The wavefront's steps (v, v+NW, ...) go two at a time: all loads of both first, then each is
  // parked in LDS and multiplied.  The very last step may be the one that K cuts: lanes past K read
  // the row's first piece instead and park zeros.
  const int steps = (K + 63) / 64;
  int count = wave < steps ? (steps - wave + NW - 1) / NW : 0;
  int k0 = wave * 64;
  auto group = [&](auto gc, auto lastc) {
    constexpr int G = decltype(gc)::value;
    constexpr bool LAST = decltype(lastc)::value;
    uint4 av[G][AL], wv[G][WL];
    bool kin = true;
#pragma unroll
    for (int u = 0; u < G; ++u) {
      int kk = k0 + u * NW * 64;
      if (LAST && u == G - 1) {
        kin = kk + lc < K;
        kk = kin ? kk : -lc;
      }
#pragma unroll
      for (int i = 0; i < AL; ++i) av[u][i] = load16(pa[i] + kk);
#pragma unroll
      for (int i = 0; i < WL; ++i) wv[u][i] = load16(pw[i] + kk);
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
#pragma unroll
      for (int i = 0; i < AL; ++i) *(uint4*)&mine[(i * 8 + lr) * SK_LD + lc] = av[u][i];
#pragma unroll
      for (int i = 0; i < WL; ++i) *(uint4*)&mine[(AR + i * 8 + lr) * SK_LD + lc] = wv[u][i];
      if (LAST && u == G - 1 && !kin) {        // past K: zeros over what the lane just parked
        const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < AL; ++i) *(uint4*)&mine[(i * 8 + lr) * SK_LD + lc] = zero;
#pragma unroll
        for (int i = 0; i < WL; ++i) *(uint4*)&mine[(AR + i * 8 + lr) * SK_LD + lc] = zero;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#pragma unroll
      for (int c = 0; c < 64; c += 32) {
        const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, *(const uint4*)&mine[(AR + fr % COLS) * SK_LD + c + fk]);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const bf16x8_t af = __builtin_bit_cast(bf16x8_t, *(const uint4*)&mine[(i * 16 + fr) * SK_LD + c + fk]);
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, wf, acc[i], 0, 0, 0);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
    k0 += G * NW * 64;
    count -= G;
  };
  while (count > UNROLL) group(std::integral_constant<int, UNROLL>{}, std::false_type{});
  switch (count) {
    case 4: if (UNROLL >= 4) group(std::integral_constant<int, (UNROLL >= 4 ? 4 : 1)>{}, std::true_type{}); break;
    case 3: if (UNROLL >= 3) group(std::integral_constant<int, (UNROLL >= 3 ? 3 : 1)>{}, std::true_type{}); break;
    case 2: if (UNROLL >= 2) group(std::integral_constant<int, (UNROLL >= 2 ? 2 : 1)>{}, std::true_type{}); break;
    case 1: group(std::integral_constant<int, 1>{}, std::true_type{}); break;
    default: break;
  }
  lds_barrier();
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (COLS == 16 || fr < COLS) red[wave][i * 16 + 4 * (lane / 16) + r][fr] = acc[i][r];
  lds_barrier();
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = t + j * NW * 64, ml = e / COLS, m = r0 + ml, c = e % COLS, n = n0 + c;
    if (e < AR * COLS && m < M && n < N) {
      float v = red[0][ml][c];
#pragma unroll
      for (int v2 = 1; v2 < NW; ++v2) v += red[v2][ml][c];
      const float e_bias = !ep.bias ? 0.f : (bias_bf16 ? __uint_as_float(e_braw[j] << 16) : __uint_as_float(e_braw[j]));
      v = ep.out_dtype == DA_BF16 ? apply_act_bf16(v + e_bias, ep.act) : apply_act(v + e_bias, ep.act);
      const size_t o = (size_t)m * ep.ldo + n;
      if (ep.accumulate) ((float*)ep.out)[o] = e_old[j] + v;
      else if (ep.out_dtype == DA_BF16) ((bf16_t*)ep.out)[o] = f32_to_bf16(v);
      else ((float*)ep.out)[o] = v;
      if (kv.cache && n >= kv.q_cols && e_slot[j] >= 0) kv_scatter_store(kv, e_slot[j], n, v);
    }
  }
}

template <int NW>
static int launch_skinny(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw,
                         const Epilogue& ep, const KvScatter& kv, int M, int N, int K) {
  const dim3 block(NW * 64);
  int mt = da_ceil_div(M, 16);
#define DA_SK_GO(AL, COLS, U) hipLaunchKernelGGL((gemm_skinny_kernel<AL, COLS, NW, U>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K)
  if (mt == 1 && NW != 4 && da_ceil_div(N, 16) < 128) {
    // few columns and one row tile: 8 columns a workgroup
    const dim3 grid(da_ceil_div(N, 8));
    if (M <= 8) DA_SK_GO(1, 8, 4); else DA_SK_GO(2, 8, 4);
    return 0;
  }
  dim3 grid(da_ceil_div(N, 16));
  // With few columns the row tiles are spread over more workgroups (blockIdx.y), as long as the chip
  // is not full: each then reads fewer rows of a.  A row's sums do not depend on it.
  for (int mb = 1; mb < mt; mb *= 2)
    if ((long)grid.x * da_ceil_div(mt, mb) <= 256) {
      grid.y = da_ceil_div(mt, mb);
      mt = mb;
      break;
    }
  // Three or four row tiles take the LDS of a compute unit for one workgroup; with somewhat more
  // workgroups than compute units a second, mostly empty round then waits for the first.  Two workgroups
  // of two row tiles share a compute unit and run side by side (GPT-2 1.5B sizes, 48 and 64 rows: 4 and
  // 2 % of a decode step).
  if (grid.y == 1 && mt >= 3 && grid.x > 256 && grid.x <= 512) {
    grid.y = 2;
    mt = 2;
  }
  DA_REQUIRE(mt >= 1 && mt <= 4, "gemm_bf16: %d row tiles", mt);
  // steps in flight: 16 to 20 loads of 16 bytes a lane
  if (mt == 1 && M <= 8) DA_SK_GO(1, 16, 4);
  else if (mt == 1) DA_SK_GO(2, 16, 4);
  else if (mt == 2) DA_SK_GO(4, 16, 3);
  else if (mt == 3) DA_SK_GO(6, 16, 2);
  else DA_SK_GO(8, 16, 2);
#undef DA_SK_GO
  return 0;
}

// ---------------------------------------------------------------------------------------------
// M <= 4 and up to 2,048 columns (a decode step of a few requests).  MFMA 4x4x4: 16 independent 4x4
// products of depth 4 a wavefront.  Lane l gives row (a) /
// column (b) l % 4 of product l / 4 and 4 consecutive k; it receives column l % 4 of that product,
// rows 0..3.  The 16 products of a step take 16 consecutive pieces of k of 8 elements (two
// instructions each), so a lane loads 16 bytes and the 16 lanes of one row of w read 256 consecutive
// bytes: whole cache lines without a detour through LDS.  A workgroup owns 4 * NG columns; wavefront v of NW takes
// the steps v, v+NW, ... of 128 elements of k; the products of a wavefront are summed over its 16
// lanes-groups at the end (two lane rotations, then LDS) in a fixed order.
// ---------------------------------------------------------------------------------------------
template <int NG, int NW, int UNROLL>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny4_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                    Epilogue ep, KvScatter kv, int M, int N, int K) {
  constexpr int MG = 1;                        // row groups of 4 (from 5 rows on gemm_skinny is faster)
  constexpr int ROWS = MG * 4, COLS = NG * 4;
  __shared__ __attribute__((aligned(16))) float red[4 * NW][COLS][ROWS];
  static_assert(NW * 64 >= 4 * ROWS * COLS, "four threads an output element");
  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int n0 = blockIdx.x * COLS;
  const int q = lane % 4, kb = (lane / 4) * 8;
  const bf16_t* wp[NG];
  const bf16_t* ap[MG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int n = n0 + g * 4 + q;
    wp[g] = w + (size_t)(n < N ? n : 0) * ldw + kb;
  }
#pragma unroll
  for (int g = 0; g < MG; ++g) {
    const int m = g * 4 + q;
    ap[g] = a + (size_t)(m < M ? m : 0) * lda + kb;
  }
  // what the epilogue needs is asked for first, as raw bits from places that always exist
  // Four threads an output element (the host launches 4 * ROWS * COLS threads at least): each sums
  // a quarter of the partial sums, the first of them stores.
  const int e_id = t / 4, e_q = t % 4;
  const int e_m = e_id / COLS, e_c = e_id % COLS, e_n = n0 + e_c;
  const bool e_ok = e_id < ROWS * COLS && e_m < M && e_n < N;
  const bool e_st = e_ok && e_q == 0;
  const bool bias_bf16 = ep.bias_dtype == DA_BF16;
  const void* e_bsrc = (e_st && ep.bias) ? ep.bias : (const void*)w;
  const int e_bidx = (e_st && ep.bias) ? e_n : 0;
  const uint32_t e_braw = bias_bf16 ? (uint32_t)((const bf16_t*)e_bsrc)[e_bidx] : ((const uint32_t*)e_bsrc)[e_bidx];
  const float e_old = *((e_st && ep.accumulate) ? (const float*)ep.out + (size_t)e_m * ep.ldo + e_n : (const float*)w);
  const int e_slot = *((e_st && kv.cache) ? kv.slot_map + e_m : (const int*)w);

  floatx4 acc[MG][NG];
#pragma unroll
  for (int i = 0; i < MG; ++i)
#pragma unroll
    for (int j = 0; j < NG; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  // The wavefront's steps go in groups of UNROLL and one last group of what is left: a group is
  // nothing but its loads, all in flight at once, and then its products.  The last step of the last
  // group may be the one that K cuts: lanes past K read the row's first piece instead and give
  // zeros for a (a multiple of 8 elements is in or out as a whole).
  const int steps = (K + 127) / 128;
  int count = wave < steps ? (steps - wave + NW - 1) / NW : 0;
  int k0 = wave * 128;
  auto group = [&](auto gc, auto lastc) {
    constexpr int G = decltype(gc)::value;
    constexpr bool LAST = decltype(lastc)::value;
    uint4 av[G][MG], wv[G][NG];
    bool kin = true;
#pragma unroll
    for (int u = 0; u < G; ++u) {
      int kk = k0 + u * NW * 128;
      if (LAST && u == G - 1) {
        kin = kk + kb < K;
        kk = kin ? kk : -kb;
      }
#pragma unroll
      for (int i = 0; i < MG; ++i) av[u][i] = load16(ap[i] + kk);
#pragma unroll
      for (int j = 0; j < NG; ++j) wv[u][j] = load16(wp[j] + kk);
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
      if (LAST && u == G - 1) {
#pragma unroll
        for (int i = 0; i < MG; ++i)
          if (!kin) av[u][i] = make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < MG; ++i)
#pragma unroll
        for (int j = 0; j < NG; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
              __builtin_bit_cast(bf16x4s_t, make_uint2(av[u][i].x, av[u][i].y)),
              __builtin_bit_cast(bf16x4s_t, make_uint2(wv[u][j].x, wv[u][j].y)), acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
              __builtin_bit_cast(bf16x4s_t, make_uint2(av[u][i].z, av[u][i].w)),
              __builtin_bit_cast(bf16x4s_t, make_uint2(wv[u][j].z, wv[u][j].w)), acc[i][j], 0, 0, 0);
        }
    }
    k0 += G * NW * 128;
    count -= G;
  };
  while (count > UNROLL) group(std::integral_constant<int, UNROLL>{}, std::false_type{});
  switch (count) {
    case 4: if (UNROLL >= 4) group(std::integral_constant<int, (UNROLL >= 4 ? 4 : 1)>{}, std::true_type{}); break;
    case 3: if (UNROLL >= 3) group(std::integral_constant<int, (UNROLL >= 3 ? 3 : 1)>{}, std::true_type{}); break;
    case 2: if (UNROLL >= 2) group(std::integral_constant<int, (UNROLL >= 2 ? 2 : 1)>{}, std::true_type{}); break;
    case 1: group(std::integral_constant<int, 1>{}, std::true_type{}); break;
    default: break;
  }
  // sum over the four products of a row of 16 lanes, then one partial a row of lanes goes to LDS
#pragma unroll
  for (int i = 0; i < MG; ++i)
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      floatx4 v = acc[i][j];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] += dpp_move<0x124, 0xF>(v[r], v[r]);      // row_ror:4
        v[r] += dpp_move<0x128, 0xF>(v[r], v[r]);      // row_ror:8
      }
      if (lane % 16 < 4) *(floatx4*)&red[wave * 4 + lane / 16][j * 4 + q][i * 4] = v;
    }
  lds_barrier();
  if (e_id < ROWS * COLS) {               // whole quads
    // thread e_q of the four takes the partial sums e_q, e_q + 4, ...: one of each wavefront
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) v += red[e_q + 4 * i][e_c][e_m];
    v += dpp_move<0xB1, 0xF>(v, v);
    v += dpp_move<0x4E, 0xF>(v, v);
    if (e_st) {
      const float e_bias = !ep.bias ? 0.f : (bias_bf16 ? __uint_as_float(e_braw << 16) : __uint_as_float(e_braw));
      v = ep.out_dtype == DA_BF16 ? apply_act_bf16(v + e_bias, ep.act) : apply_act(v + e_bias, ep.act);
      const size_t o = (size_t)e_m * ep.ldo + e_n;
      if (ep.accumulate) ((float*)ep.out)[o] = e_old + v;
      else if (ep.out_dtype == DA_BF16) ((bf16_t*)ep.out)[o] = f32_to_bf16(v);
      else ((float*)ep.out)[o] = v;
      if (kv.cache && e_n >= kv.q_cols && e_slot >= 0) kv_scatter_store(kv, e_slot, e_n, v);
    }
  }
}

template <int NG>
static int launch_skinny4(int nw, hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw,
                          const Epilogue& ep, const KvScatter& kv, int M, int N, int K) {
  DA_REQUIRE(M <= 4, "gemm_bf16: %d rows for one group of 4", M);
  const dim3 grid(da_ceil_div(N, NG * 4));
  if (nw == 16) hipLaunchKernelGGL((gemm_skinny4_kernel<NG, 16, 4>), grid, dim3(1024), 0, s, A, lda, W, ldw, ep, kv, M, N, K);
  else if (nw == 8) hipLaunchKernelGGL((gemm_skinny4_kernel<NG, 8, 4>), grid, dim3(512), 0, s, A, lda, W, ldw, ep, kv, M, N, K);
  else hipLaunchKernelGGL((gemm_skinny4_kernel<NG, 4, 4>), grid, dim3(256), 0, s, A, lda, W, ldw, ep, kv, M, N, K);
  return 0;
}

extern "C" int da_gemm_bf16(const void* a, int lda, const void* w, int ldw, const void* bias, int bias_dtype,
                            int act, int accumulate, void* out, int out_dtype, int ldo, int M, int N, int K,
                            void* kv_cache, const int* slot_map, int q_cols, int kv_cols, int Hkv, int D, int page,
                            void* stream) {
  DA_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  DA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0,
             "gemm_bf16: K, lda and ldw must be multiples of 8 (K=%d lda=%d ldw=%d)", K, lda, ldw);
  DA_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  DA_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_bf16: leading sizes too small");
  DA_REQUIRE(!accumulate || out_dtype == DA_F32, "gemm_bf16: accumulation needs a 32-bit output");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_SILU, "gemm_bf16: unknown activation %d", act);
  if (kv_cache) {
    DA_REQUIRE(out_dtype == DA_BF16 && !accumulate && q_cols >= 0 && kv_cols == Hkv * D && q_cols + 2 * kv_cols == N &&
               page > 0 && (page & (page - 1)) == 0, "gemm_bf16: the q|k|v columns (%d + 2*%d) must add up to N=%d, the page size a power of two", q_cols, kv_cols, N);
  }
  if (M == 0) return 0;
  Epilogue ep{bias, bias_dtype, act, accumulate, out, out_dtype, ldo};
  KvScatter kv{kv_cache, slot_map, q_cols, kv_cols, Hkv, D, page};
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  if (M <= 4 && N <= 2048) {
    // Measured: up to 4 rows and 2,048 columns the 4x4x4 form is ahead, by 20 to 25 % with K from 2,048 on.
    const int nw = K >= 2048 ? 16 : (K >= 1024 ? 8 : 4);   // by K alone, so a row's sums keep their order
    if (N <= 1024 ? launch_skinny4<1>(nw, s, A, lda, W, ldw, ep, kv, M, N, K)
                  : launch_skinny4<2>(nw, s, A, lda, W, ldw, ep, kv, M, N, K)) return 1;
  } else if (M <= 32 || (M <= 64 && N <= 8192)) {     // (a vocabulary with more than 32 rows: block tiles reuse the rows of a)
    // The number of wavefronts that split K depends on K and N alone, so a row's sums keep their order:
    // 4 where the workgroups are many (a vocabulary: several then share a compute unit), else 8, or 12 for a long K.
    const int nw = da_ceil_div(N, 16) > 1024 ? 4 : (K >= 2048 ? 12 : 8);
    if (nw == 4 ? launch_skinny<4>(s, A, lda, W, ldw, ep, kv, M, N, K)
                : (nw == 8 ? launch_skinny<8>(s, A, lda, W, ldw, ep, kv, M, N, K)
                           : launch_skinny<12>(s, A, lda, W, ldw, ep, kv, M, N, K))) return 1;
  } else {
    // Smaller tiles where larger ones would leave compute units idle (measured on GPT-2's shapes).
    // Every configuration sums a row's products in the same order (64-wide slabs, 16 at a time), so
    // the choice does not change a result.
    const int wide = da_gemm_wide_takes(act, accumulate, out_dtype, K) ? da_gemm_wide_choice(M, N, K) : DA_WIDE_NONE;
    if (wide != DA_WIDE_NONE) {
      // operands straight into LDS where such tiles fill the chip: the same sums in the same order, less LDS traffic
      da_gemm_wide_launch(s, A, lda, W, ldw, ep, kv, M, N, K, wide);
      DA_CHECK_LAUNCH("gemm_bf16");
      return 0;
    }
    const long tiles128 = (long)da_ceil_div(M, 128) * da_ceil_div(N, 128);
    const long tiles12864 = (long)da_ceil_div(M, 128) * da_ceil_div(N, 64);
    // (up to 256 tiles a workgroup has its compute unit to itself: four slabs in flight instead of two, with the
    // registers that a second workgroup would have needed: GPT-2 1.5B's proj and out-proj, 3.6 % of its prefill)
    if (tiles128 >= 192 && tiles128 <= 256) launch_tile<128, 128, 4, 2, 4>(s, A, lda, W, ldw, ep, kv, M, N, K);
    else if (tiles128 >= 192) launch_tile<128, 128, 4, 2, 2>(s, A, lda, W, ldw, ep, kv, M, N, K);
    else if (tiles12864 >= 192) launch_tile<128, 64, 4, 2, 4>(s, A, lda, W, ldw, ep, kv, M, N, K);
    else launch_tile<64, 64, 2, 2, 4>(s, A, lda, W, ldw, ep, kv, M, N, K);
  }
  DA_CHECK_LAUNCH("gemm_bf16");
  return 0;
}
