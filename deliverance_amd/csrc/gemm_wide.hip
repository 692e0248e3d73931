// The block-tile product for large steps: operands from memory straight into LDS.
//
//   out[m, n] (+)= act( sum_k a[m, k] * w[n, k] + bias[n] )        (a [M, K], w [N, K], bfloat16, K contiguous)
//
// The first shape: tiles of 256 x 256, eight wavefronts, two a SIMD, each with 128 x 64 of the tile (4 x 2
// products of 32 x 32 x 16, 128 accumulation registers): a k-step of 16 takes 6 fragment reads for 8 matrix
// instructions, half the LDS traffic a flop of the 128 x 128 tile kernel (gemm_mfma.hip), whose matrix cores
// wait for LDS most of the time.  Two smaller shapes for products whose 256 x 256 tiles would leave compute
// units idle, both with eight wavefronts: 256 x 128 (64 x 64 a wavefront: 4 reads for 4 matrix instructions),
// and 128 x 128 (32 x 64 a wavefront), of which two workgroups share a compute unit (da_gemm_wide_choice).
// A slab of 64 elements of k is 128 bytes a row, one cache line: it goes from memory into LDS
// without passing registers (da_lds_dma.h), into one of two stages for a (one slab ahead of the
// products) and one of three for w (two slabs ahead: weights come from memory, not from a cache); one
// barrier a slab.  Rows lie unpadded in LDS (a copy writes 1,024 consecutive bytes: 8 rows); the
// 16-byte pieces of row r are stored at position piece ^ (r % 8), which the copy does by choosing what
// each lane fetches, so that the fragment reads of 16 consecutive rows spread over all banks.
// Fragments are read one k-step ahead of the products that use them.
//
// An output element sums over k in ascending steps of 16 like the other tile forms: the result has the
// same bits.  K must be a multiple of 64 (other sizes go to gemm_mfma.hip's kernels).
//
// The epilogue is per wavefront: 32 rows x 64 columns at a time are parked in the wavefront's own piece
// of LDS (bias and activation applied, rounded to the output's type), and leave in 16-byte pieces, whole
// rows side by side; += adds to 16-byte pieces read the same way; a fused q|k|v projection also writes
// its k and v columns to the rows' places in the paged cache (keys in 16-byte pieces of their rows,
// values in 16-byte runs where 8 rows' places are consecutive).
#include "gemm_common.h"
#include <da_lds_dma.h>
#include <type_traits>

#define WD_BK 64
#define WD_ROW_BYTES (WD_BK * 2)
#define WD_REGION_BYTES 8960          // a wavefront's piece of LDS in the epilogue: 32 x 68 floats, then 32 places

__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// OUTMODE: 0 bf16 store, 1 f32 store, 2 f32 +=
template <int TM, int TN, int ACT, int OUTMODE>
__device__ __forceinline__ void
wide_epilogue(floatx16 (&acc)[TM][TN], const float (&bias)[TN], char* region, const void* safe, const Epilogue& ep,
              const KvScatter& kv, int M, int N, int mw, int nw, int lane) {
  constexpr int WC = 32 * TN;                                   // the wavefront's columns
  constexpr int ES = OUTMODE == 0 ? 2 : 4, CH = 16 / ES;       // bytes an element; elements a 16-byte piece
  constexpr int LDT = WC + CH;                                  // a parked row, padded by one piece
  constexpr int CPR = WC / CH, NCHK = 32 * CPR / 64;            // pieces a row; pieces a lane and pass
  static_assert(32 * LDT * ES + 32 * 4 <= WD_REGION_BYTES, "a wavefront's epilogue region");
  const int fr = lane % 32;
  int* slots = (int*)(region + 32 * LDT * ES);
  const bool wide = (uintptr_t)ep.out % 16 == 0 && ep.ldo % CH == 0;
  // A q|k|v product's cache write: what does not change from pass to pass.  The page size is a power of two
  // (checked on the host): places split into page and row by shift and mask.
  const int lgp = kv.cache ? 31 - __builtin_clz(kv.page) : 0, pmask = kv.page - 1;
  const int v0 = kv.q_cols + kv.kv_cols;                        // the first value column
  const bool kwide = kv.cache && (uintptr_t)kv.cache % 16 == 0 && kv.D % 8 == 0 && kv.q_cols % 8 == 0;
  const bool vwide = kv.cache && (uintptr_t)kv.cache % 8 == 0 && kv.page % 4 == 0;
  const long long page_stride = 2LL * kv.Hkv * kv.page * kv.D;
  int kh[NCHK], kd[NCHK];                                       // head and dimension of a key piece's first column
  int vcol[TN];                                                 // a value column's place in a page: its head's values, its dimension's run
  if (OUTMODE == 0 && kv.cache) {
#pragma unroll
    for (int k = 0; k < NCHK; ++k) {
      const int c2 = nw + ((lane + 64 * k) % CPR) * CH - kv.q_cols, cs = c2 > 0 ? c2 : 0;
      kh[k] = cs / kv.D;
      kd[k] = cs % kv.D;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int cc = nw + j * 32 + fr - v0, cs = cc > 0 ? cc : 0;
      vcol[j] = (kv.Hkv + cs / kv.D) * kv.page * kv.D + (cs % kv.D) * kv.page;
    }
  }
  // (a pass per constant i: an index that is not a constant would put the accumulators into memory)
  auto pass = [&](auto ic) {
    constexpr int i = decltype(ic)::value;
    const int mp = mw + i * 32;                                 // the pass's first row
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ml = 8 * (r / 4) + 4 * (lane / 32) + (r % 4), nl = j * 32 + fr;
        if (OUTMODE == 0) ((bf16_t*)region)[ml * LDT + nl] = f32_to_bf16(apply_act_bf16(acc[i][j][r] + bias[j], ACT));
        else ((float*)region)[ml * LDT + nl] = apply_act(acc[i][j][r] + bias[j], ACT);
      }
    if (OUTMODE == 0 && kv.cache && lane < 32) slots[lane] = mp + lane < M ? kv.slot_map[mp + lane] : -1;
    wave_lds_sync();

    uint4 val[NCHK];
    int mm[NCHK], nn[NCHK];
#pragma unroll
    for (int k = 0; k < NCHK; ++k) {
      const int q = lane + 64 * k, row = q / CPR, c = q % CPR;
      mm[k] = mp + row;
      nn[k] = nw + c * CH;
      val[k] = *(const uint4*)(region + (size_t)(row * LDT + c * CH) * ES);
    }
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
    // (for +=, such a piece still holds the bare products here: only whole pieces were added to above)
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

    if (OUTMODE == 0 && kv.cache) {
      // keys: eight dimensions of one key are one piece of its cache row (head and dimension of a piece's
      // columns were worked out before the passes)
#pragma unroll
      for (int k = 0; k < NCHK; ++k) {
        const int slot = slots[mm[k] - mp];
        if (slot < 0 || nn[k] >= N || nn[k] + 8 <= kv.q_cols || nn[k] >= v0) continue;
        const int pg = slot >> lgp, prow = slot & pmask;
        if (kwide) {
          *(uint4*)((bf16_t*)kv.cache + cache_k_row(pg, kh[k], prow, kv.Hkv, kv.page, kv.D) + kd[k]) = val[k];
          continue;
        }
        const uint32_t words[4] = {val[k].x, val[k].y, val[k].z, val[k].w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (nn[k] + e >= kv.q_cols && nn[k] + e < v0)
            kv_scatter_bits(kv, pg, prow, nn[k] + e, (bf16_t)(words[e / 2] >> (16 * (e % 2))));
      }
      // values, straight from the accumulators: a lane holds 4 consecutive rows of its column (r % 4), which
      // are 8 consecutive bytes of the dimension-major page when the rows' places are 4 consecutive ones from
      // a multiple of 4 on (a prompt portion's are); the lane of the other half holds the 4 rows beside them
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = nw + j * 32 + fr;
        if (n < v0 || n >= N) continue;
        bf16_t* vb = (bf16_t*)kv.cache;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int r0 = 8 * q + 4 * (lane / 32);             // the first of the lane's 4 rows in this pass
          const uint4 su = *(const uint4*)&slots[r0];
          const struct { int x, y, z, w; } sl = {(int)su.x, (int)su.y, (int)su.z, (int)su.w};
          uint32_t w2[2];
#pragma unroll
          for (int e = 0; e < 2; ++e)
            w2[e] = pack2_bf16(apply_act_bf16(acc[i][j][4 * q + 2 * e] + bias[j], ACT),
                               apply_act_bf16(acc[i][j][4 * q + 2 * e + 1] + bias[j], ACT));
          const bool run = vwide && sl.x >= 0 && (sl.x & 3) == 0 && sl.y == sl.x + 1 && sl.z == sl.x + 2 && sl.w == sl.x + 3;
          if (run) {
            *(uint2*)(vb + (long long)(sl.x >> lgp) * page_stride + vcol[j] + (sl.x & pmask)) = make_uint2(w2[0], w2[1]);
            continue;
          }
          const int s4[4] = {sl.x, sl.y, sl.z, sl.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (s4[e] >= 0)
              vb[(long long)(s4[e] >> lgp) * page_stride + vcol[j] + (s4[e] & pmask)] = (bf16_t)(w2[e / 2] >> (16 * (e % 2)));
        }
      }
    }
    wave_lds_sync();       // the next pass parks over what this one read
  };
  pass(std::integral_constant<int, 0>{});
  if (TM > 1) pass(std::integral_constant<int, (TM > 1 ? 1 : 0)>{});
  if (TM > 2) pass(std::integral_constant<int, (TM > 2 ? 2 : 0)>{});
  if (TM > 3) pass(std::integral_constant<int, (TM > 3 ? 3 : 0)>{});
}

// BM x BN: the tile; WM x WN wavefronts of (BM / WM) x (BN / WN) each.  In use: 256 x 256 with 2 x 4
// wavefronts of 128 x 64, one workgroup a compute unit (160 KB of LDS); 256 x 128 with 4 x 2 of 64 x 64
// (112 KB); 128 x 128 with 4 x 2 of 32 x 64, two workgroups a compute unit (80 KB each); which of them
// for which sizes: da_gemm_wide_choice.  Measured beside them: 256 x 256 with four wavefronts of 128 x 128
// (a third less LDS traffic; 15 to 25 % slower: one wavefront a SIMD has nobody to fill its waits);
// 128 x 128 with 2 x 2 wavefronts of 64 x 64 (7 to 10 % behind the eight wavefronts at a short K).
template <int BM, int BN, int WM, int WN, int ACT, int OUTMODE>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_wide_kernel(const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w, int ldw,
                 Epilogue ep, KvScatter kv, int M, int N, int K, int tiles_m, int tiles_n) {
  // Two stages of a slab of a, three of a slab of w.  The rows of a were written by the kernel before and
  // come from a cache; w comes from memory for the first time and needs the longer way ahead.
  constexpr int A_BYTES = BM * WD_ROW_BYTES, W_BYTES = BN * WD_ROW_BYTES;      // a slab of a, of w, in LDS
  constexpr int NW = WM * WN, TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int CA = BM / 8 / NW, CW = BN / 8 / NW;                             // copies a wavefront and slab
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0 && BM % (32 * WM) == 0 && BN % (32 * WN) == 0 && NW % 2 == 0,
                "the tile does not split over the wavefronts");
  static_assert(BN / WN == 64, "the epilogue parks 64 columns a wavefront");
  __shared__ __attribute__((aligned(1024))) char smem[2 * A_BYTES + 3 * W_BYTES];
  static_assert(NW * WD_REGION_BYTES <= 2 * A_BYTES + 3 * W_BYTES, "the epilogue regions fit the stages");
  char* const smem_a = smem;
  char* const smem_w = smem + 2 * A_BYTES;

  // Each XCD (workgroups that follow each other in launch order land on different ones) takes a
  // contiguous run of tiles, m fastest, so that its workgroups share slabs of w in its L2.
  const int nblocks = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblocks / 8, rem = nblocks % 8;
    const int xcd = pid % 8, local = pid / 8;
    pid = xcd * per + (xcd < rem ? xcd : rem) + local;
  }
  const int m0 = (pid % tiles_m) * BM, n0 = (pid / tiles_m) * BN;

  const int t = threadIdx.x, lane = t % 64;
  const int wave = __builtin_amdgcn_readfirstlane(t / 64);
  const int wm = (wave % WM) * (BM / WM), wn = (wave / WM) * (BN / WN);
  const int fr = lane % 32, fk = lane / 32;

  // Copies: a stage of a (of w) is BM / 8 (BN / 8) blocks of 8 rows; wavefront v takes blocks v, v + NW, ...
  // Lane l of a copy stands for row l / 8 of the block and position l % 8 of that row, which holds the
  // row's piece (l % 8) ^ (r / 2 % 8), r the row's number in the stage.  Rows past the edge of a or w read
  // the last row: what they give is never stored.
  const bf16_t* src_a[CA];
  const bf16_t* src_w[CW];
  int blk[CA > CW ? CA : CW];                        // byte offset of the wavefront's blocks in a stage
  {
    // (row r of a stage is row l / 8 of block v + NW i, NW even: r / 2 % 8 = (4 (v % 2) + l / 16) % 8)
    const int rl = lane / 8, piece = (lane % 8) ^ ((4 * (wave & 1) + (rl >> 1)) & 7);
#pragma unroll
    for (int i = 0; i < (CA > CW ? CA : CW); ++i) {
      const int b = i * NW + wave;
      const int ra = m0 + b * 8 + rl, rw = n0 + b * 8 + rl;
      if (i < CA) src_a[i] = a + (size_t)(ra < M ? ra : M - 1) * lda + piece * 8;
      if (i < CW) src_w[i] = w + (size_t)(rw < N ? rw : N - 1) * ldw + piece * 8;
      blk[i] = b * 1024;
    }
  }
#define WD_COPY_A(i, stage) { lds_dma16(src_a[i], smem_a + (stage) * A_BYTES + blk[i]); src_a[i] += WD_BK; }
#define WD_COPY_W(i, stage) { lds_dma16(src_w[i], smem_w + (stage) * W_BYTES + blk[i]); src_w[i] += WD_BK; }

  // Fragments: lane l gives row l % 32 of a 32-row piece and the 8 k from 8 * (l / 32) of a k-step:
  // piece 2 * step + l / 32 of its row, stored at that number ^ (row / 2 % 8).
  int a_off[TM], w_off[TN], k_off[4];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_off[i] = (wm + i * 32 + fr) * WD_ROW_BYTES;
#pragma unroll
  for (int j = 0; j < TN; ++j) w_off[j] = (wn + j * 32 + fr) * WD_ROW_BYTES;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) k_off[ks] = ((2 * ks + fk) ^ ((fr >> 1) & 7)) * 16;
#define WD_READ(FA, FB, sa, sw, ks)                                                                                  \
  {                                                                                                                  \
    const char* pa = smem_a + (sa) * A_BYTES + k_off[ks];                                                            \
    const char* pw = smem_w + (sw) * W_BYTES + k_off[ks];                                                            \
    _Pragma("unroll") for (int i = 0; i < TM; ++i) FA[i] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(pa + a_off[i])); \
    _Pragma("unroll") for (int j = 0; j < TN; ++j) FB[j] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(pw + w_off[j])); \
  }
#define WD_MFMA1(FA, FB, q) \
  acc[(q) / TN][(q) % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FA[(q) / TN], FB[(q) % TN], acc[(q) / TN][(q) % TN], 0, 0, 0)
#define WD_MFMA(FA, FB) { _Pragma("unroll") for (int q = 0; q < TM * TN; ++q) WD_MFMA1(FA, FB, q); }
#define WD_FENCE() __builtin_amdgcn_sched_barrier(0)

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // The bias is asked for now, as raw bits from a place that always exists; it has long arrived when
  // the products are done.  No other ordinary load stands between here and the end of the slabs, so
  // that the copies' count of outstanding loads is exact.
  const bool bias_bf16 = ep.bias_dtype == DA_BF16;
  uint32_t braw[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn + j * 32 + fr;
    const bool has = ep.bias && n < N;
    const void* bsrc = has ? ep.bias : (const void*)w;
    const int idx = has ? n : 0;
    braw[j] = bias_bf16 ? (uint32_t)((const bf16_t*)bsrc)[idx] : ((const uint32_t*)bsrc)[idx];
  }
  float bias[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) bias[j] = !ep.bias ? 0.f : (bias_bf16 ? __uint_as_float(braw[j] << 16) : __uint_as_float(braw[j]));

  // Order of the copies: a(0) w(0) | a(1) w(1) | w(2) | then, after the barrier that ends slab s, a(s + 2)
  // and w(s + 3) into the stages that slab s left.  Copies land in the order they were asked for, so
  // "slab s + 1 is there" is "at most the four youngest copies, w(s + 2), are still under way".
  const int nslab = K / WD_BK;
  bf16x8_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];
#pragma unroll
  for (int i = 0; i < CA; ++i) WD_COPY_A(i, 0);
#pragma unroll
  for (int i = 0; i < CW; ++i) WD_COPY_W(i, 0);
  if (nslab > 1) {
#pragma unroll
    for (int i = 0; i < CA; ++i) WD_COPY_A(i, 1);
#pragma unroll
    for (int i = 0; i < CW; ++i) WD_COPY_W(i, 1);
  }
  if (nslab > 2) {
#pragma unroll
    for (int i = 0; i < CW; ++i) WD_COPY_W(i, 2);
  }
  static_assert(CA + 2 * CW <= 15, "the count of copies under way fits its field");
  if (nslab > 2) DA_WAIT_VMCNT(CA + 2 * CW); else if (nslab > 1) DA_WAIT_VMCNT(CA + CW); else DA_WAIT_VMCNT(0);
  __builtin_amdgcn_s_barrier();
  WD_READ(fa0, fb0, 0, 0, 0);
  int sw = 0;                                          // the stage of w that holds slab s
  // One slab.  COPY_A: slab s + 2 exists; COPY_W: slab s + 3 exists; NEXT: slab s + 1 exists.
  auto slab = [&](int s, auto copy_a_c, auto copy_w_c, auto next_c) {
    constexpr bool COPY_A = decltype(copy_a_c)::value, COPY_W = decltype(copy_w_c)::value, NEXT = decltype(next_c)::value;
    const int sa = s & 1, sw1 = sw == 2 ? 0 : sw + 1;
    WD_FENCE();
    // (the first product stands in front of the reads: the wait that the compiler puts before it then
    // covers the fragments it needs and nothing that was only just asked for)
    WD_MFMA1(fa0, fb0, 0);
    WD_FENCE();
    WD_READ(fa1, fb1, sa, sw, 1);
    WD_FENCE();
#pragma unroll
    for (int q = 1; q < TM * TN; ++q) WD_MFMA1(fa0, fb0, q);
    WD_FENCE();
    WD_READ(fa0, fb0, sa, sw, 2);
    WD_FENCE();
    WD_MFMA(fa1, fb1);
    WD_FENCE();
    WD_READ(fa1, fb1, sa, sw, 3);
    WD_FENCE();
    WD_MFMA(fa0, fb0);
    WD_FENCE();
    // Slab s + 1 must have landed, and every wavefront must be done reading slab s, before a(s + 2) and
    // w(s + 3) take its place: one barrier for both.
    if (COPY_A) DA_WAIT_VMCNT(CW); else DA_WAIT_VMCNT(0);     // (COPY_A: the tail before this one asked for w(s + 2) last)
    __builtin_amdgcn_s_waitcnt(0xC07F);                        // lgkmcnt(0): this wavefront's reads of slab s are complete
    __builtin_amdgcn_s_barrier();
    // The slab's last k-step, its products one by one, and between them the copies and the reads of slab
    // s + 1's first fragments: the matrix cores have work while the wavefront issues the rest.
    constexpr int CPQ = (CA + CW + TM * TN - 1) / (TM * TN);      // copies after each product
    constexpr int RPQ = (TM + TN + TM * TN - 1) / (TM * TN);      // reads after each product
#pragma unroll
    for (int q = 0; q < TM * TN; ++q) {
      WD_MFMA1(fa1, fb1, q);
#pragma unroll
      for (int c = q * CPQ; c < (q + 1) * CPQ; ++c) {             // (all of a's before all of w's)
        if (COPY_A && c < CA) WD_COPY_A(c, sa);
        if (COPY_W && c >= CA && c < CA + CW) WD_COPY_W(c - CA, sw);
      }
#pragma unroll
      for (int r = q * RPQ; r < (q + 1) * RPQ; ++r) {             // (a's fragments, then w's)
        constexpr int LAST_A = TM - 1, LAST_W = TN - 1;
        const int ia = r < TM ? r : LAST_A, iw = (r >= TM && r < TM + TN) ? r - TM : LAST_W;    // (indices that exist, whatever r)
        if (NEXT && r < TM) fa0[ia] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(smem_a + (sa ^ 1) * A_BYTES + k_off[0] + a_off[ia]));
        if (NEXT && r >= TM && r < TM + TN) fb0[iw] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(smem_w + sw1 * W_BYTES + k_off[0] + w_off[iw]));
      }
      WD_FENCE();
    }
    sw = sw1;
  };
  {
    const std::true_type yes{};
    const std::false_type no{};
    int s = 0;
    for (; s + 3 < nslab; ++s) slab(s, yes, yes, yes);
    if (s + 2 < nslab) slab(s++, yes, no, yes);
    if (s + 1 < nslab) slab(s++, no, no, yes);
    slab(s, no, no, no);
  }
#undef WD_COPY_A
#undef WD_COPY_W
#undef WD_READ
#undef WD_MFMA
#undef WD_MFMA1
#undef WD_FENCE
  // (the last barrier of the loop: nobody reads the stages any more)
  wide_epilogue<TM, TN, ACT, OUTMODE>(acc, bias, smem + wave * WD_REGION_BYTES, (const void*)w, ep, kv, M, N, m0 + wm, n0 + wn, lane);
}

template <int BM, int BN, int WM, int WN, int ACT>
static void launch_wide_act(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                            const KvScatter& kv, int M, int N, int K) {
  const int tiles_m = da_ceil_div(M, BM), tiles_n = da_ceil_div(N, BN);
  const dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  if (ep.accumulate)
    hipLaunchKernelGGL((gemm_wide_kernel<BM, BN, WM, WN, DA_ACT_NONE, 2>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
  else if (ep.out_dtype == DA_F32)
    hipLaunchKernelGGL((gemm_wide_kernel<BM, BN, WM, WN, DA_ACT_NONE, 1>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((gemm_wide_kernel<BM, BN, WM, WN, ACT, 0>), grid, block, 0, s, A, lda, W, ldw, ep, kv, M, N, K, tiles_m, tiles_n);
}

template <int BM, int BN, int WM, int WN>
static void launch_wide(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                        const KvScatter& kv, int M, int N, int K) {
  switch (ep.act) {
    case DA_ACT_GELU_TANH: launch_wide_act<BM, BN, WM, WN, DA_ACT_GELU_TANH>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_GELU_ERF: launch_wide_act<BM, BN, WM, WN, DA_ACT_GELU_ERF>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_RELU: launch_wide_act<BM, BN, WM, WN, DA_ACT_RELU>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    case DA_ACT_SILU: launch_wide_act<BM, BN, WM, WN, DA_ACT_SILU>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
    default: launch_wide_act<BM, BN, WM, WN, DA_ACT_NONE>(s, A, lda, W, ldw, ep, kv, M, N, K); break;
  }
}

// What these tiles take: K in whole slabs, and an activation only with a bfloat16 result (the forms
// that a model's layers use; everything else stays with gemm_mfma.hip's tiles).
bool da_gemm_wide_takes(int act, int accumulate, int out_dtype, int K) {
  return K % WD_BK == 0 && K >= WD_BK && (act == DA_ACT_NONE || (!accumulate && out_dtype == DA_BF16));
}

// Which shape of tile pays, if any (DA_WIDE_NONE: gemm_mfma.hip's tiles).  A tile is a compute unit's
// work for the whole product, so the tiles must fill most of the last round of 256 compute units.
// Measured on MI355X with 512 to 8,192 rows, N from 768 to 6,400, K from 768 to 6,400, stores and +=:
//  - 256 x 256 where its tiles fill 55 % of their last round: ahead of the 128 x 128 tiles from 152 tiles on
//    (2,048 rows, N = 4,800: 39 against 47 us; N = 6,400, 200 tiles: 42 against 62 us), behind at 128 tiles
//    and fewer (N = 4,096: 30 against 27 us);
//  - else, where 128 x 128 tiles would be 257 to 512, so that some compute units had two of gemm_mfma.hip's
//    and others one: up to a K of 2,048 tiles of 256 x 128, one a compute unit (2,048 rows: N = 2,304,
//    K = 768 16.2 against 18.9 us; N = 3,072, K = 1,024 20.3 against 23.3; 1,536 rows, N = 4,800, K = 1,600
//    28.8 against 35.3); beyond, 128 x 128, two a compute unit (4,096 rows, N = 1,600, K = 6,400, += 113
//    against 130 us; 8,192 rows, N = 768, K = 3,072 58 against 69);
//  - where they would be 140 to 256, one a compute unit: 128 x 128 up to a K of 4,096 (1,024 rows, N = 2,304
//    10.6 against 13.5 us; 512 rows, N = 4,800 16.7 against 22.3; 2,048 rows, N = K = 1,600, += 21.1 against
//    23.3; 4,096 rows, N = 1,024, K = 4,096 48.6 against 56.4); beyond, the four slabs in flight of
//    gemm_mfma.hip's tiles win (2,048 rows, N = 1,600, K = 6,400: 65 against 79 us).
int da_gemm_wide_choice(int M, int N, int K) {
  const long tiles = (long)da_ceil_div(M, 256) * da_ceil_div(N, 256);
  const long rounds = (tiles + 255) / 256;
  if (tiles * 100 >= rounds * 256 * 55) return DA_WIDE_256x256;
  const long tiles128 = (long)da_ceil_div(M, 128) * da_ceil_div(N, 128);
  if (tiles128 > 256 && tiles128 <= 512) return K <= 2048 ? DA_WIDE_256x128 : DA_WIDE_128x128;
  if (tiles128 >= 140 && tiles128 <= 256 && K <= 4096) return DA_WIDE_128x128;
  return DA_WIDE_NONE;
}

void da_gemm_wide_launch(hipStream_t s, const bf16_t* A, int lda, const bf16_t* W, int ldw, const Epilogue& ep,
                         const KvScatter& kv, int M, int N, int K, int shape) {
  if (shape == DA_WIDE_128x128) launch_wide<128, 128, 4, 2>(s, A, lda, W, ldw, ep, kv, M, N, K);
  else if (shape == DA_WIDE_256x128) launch_wide<256, 128, 4, 2>(s, A, lda, W, ldw, ep, kv, M, N, K);
  else launch_wide<256, 256, 2, 4>(s, A, lda, W, ldw, ep, kv, M, N, K);
}

// These tiles alone, of the shape asked for (DA_WIDE_256x256, DA_WIDE_256x128, DA_WIDE_128x128), whatever the
// product's sizes (tests and timing call it; da_gemm_bf16 chooses by them).
extern "C" int da_gemm_bf16_wide(const void* a, int lda, const void* w, int ldw, const void* bias, int bias_dtype,
                                 int act, int accumulate, void* out, int out_dtype, int ldo, int M, int N, int K,
                                 void* kv_cache, const int* slot_map, int q_cols, int kv_cols, int Hkv, int D, int page,
                                 int shape, void* stream) {
  DA_REQUIRE(shape >= DA_WIDE_256x256 && shape <= DA_WIDE_128x128, "gemm_bf16_wide: unknown tile shape %d", shape);
  DA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16_wide: bad sizes M=%d N=%d K=%d", M, N, K);
  DA_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldo >= N, "gemm_bf16_wide: leading sizes (lda=%d ldw=%d ldo=%d)", lda, ldw, ldo);
  DA_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16_wide: operands must be 16-byte aligned");
  DA_REQUIRE(!accumulate || out_dtype == DA_F32, "gemm_bf16_wide: accumulation needs a 32-bit output");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_SILU, "gemm_bf16_wide: unknown activation %d", act);
  DA_REQUIRE(da_gemm_wide_takes(act, accumulate, out_dtype, K),
             "gemm_bf16_wide: K=%d must be a multiple of %d, and an activation goes with a bfloat16 result", K, WD_BK);
  if (kv_cache) {
    DA_REQUIRE(out_dtype == DA_BF16 && !accumulate && q_cols >= 0 && kv_cols == Hkv * D && q_cols + 2 * kv_cols == N &&
               page > 0 && (page & (page - 1)) == 0, "gemm_bf16_wide: the q|k|v columns (%d + 2*%d) must add up to N=%d, the page size a power of two", q_cols, kv_cols, N);
  }
  Epilogue ep{bias, bias_dtype, act, accumulate, out, out_dtype, ldo};
  KvScatter kv{kv_cache, slot_map, q_cols, kv_cols, Hkv, D, page};
  da_gemm_wide_launch((hipStream_t)stream, (const bf16_t*)a, lda, (const bf16_t*)w, ldw, ep, kv, M, N, K, shape);
  DA_CHECK_LAUNCH("gemm_bf16_wide");
  return 0;
}
