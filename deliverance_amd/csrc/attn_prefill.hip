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
//
// Few workgroups (a prompt of a thousand tokens and a dozen heads gives fewer than the chip has
// compute units, and the one with the last rows walks all keys alone): the wavefronts of a
// workgroup then also share out the keys.  RB row blocks of 32 x KP key phases: a round parks KP
// consecutive tiles in KP LDS buffers, wavefront (row block, phase k) multiplies tile k of the round,
// and at the end the phases' partial results (maximum, sum of weights, weighted sum) are merged in
// LDS in the order of the phases.  A tile's phase is (first key / 64) mod KP, whatever the workgroup:
// a row's sums still depend on its position, the window and KP only; RB x KP is chosen from the
// step's shape on the host.  Smaller row blocks are for short portions only: every row block of 32
// reads its keys anew, and on long prompts that traffic, not the longest workgroup, binds.
#include "common.h"
#include <da_lane_swap.h>
#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define PF_BK 64           // keys per tile
#define PF_VLD (PF_BK + 8) // padded length of a value row in LDS
#define PF_BT_MAX 2048      // block-table entries a workgroup keeps in LDS (more are read from memory)
#define PF_BT_MAX_PHASED 512   // ... where key phases need the LDS for their tiles
#define PF_PHASED_MAX_WORKGROUPS 256   // 128-row workgroups up to which eight wavefronts (4 x 2) are ahead of four: one a compute unit

// head size / 16; wavefronts (32 query rows each) per workgroup; whether the block table's entries
// for the workgroup's keys fit its LDS copy (a table entry read from memory in front of a tile's loads
// makes them wait for it, and for every load still in flight)
template <int D16, int RB, int KP, bool BT_LDS>
// (head sizes up to 64 with four wavefronts: registers held to 256, so that two workgroups share a compute unit)
__global__ void __launch_bounds__(RB * KP * DA_WAVE, (RB * KP == 4 && D16 <= 4) ? 2 : 1)
attn_prefill_kernel(const bf16_t* __restrict__ q, int q_ld, const bf16_t* __restrict__ cache,
                    const int* __restrict__ block_table, int max_blocks,
                    const int* __restrict__ q_start, const int* __restrict__ seq_lens, int seq0,
                    int Hq, int Hkv, int page, float scale, int window,
                    bf16_t* __restrict__ out, int out_ld) {
  constexpr int D = D16 * 16;
  constexpr int DT = (D + 31) / 32;       // 32-dimension tiles of the output
  constexpr int KLD = D + 8;              // padded length of a key row in LDS
  constexpr int PF_WAVES = RB * KP;
  constexpr int PF_BQ = RB * 32;          // query rows per workgroup
  constexpr int THREADS = PF_WAVES * DA_WAVE;
  // one phase: two buffers, a tile is multiplied out of one while the next is parked in the other;
  // KP phases: the KP tiles of a round
  constexpr int NB = KP == 1 ? 2 : KP;
  constexpr int RT = KP == 1 ? 1 : KP;    // tiles that one fetch asks for
  constexpr int K_PIECES = RT * PF_BK * (D / 8), V_PIECES = RT * DT * 32 * (PF_BK / 8);   // 16-byte pieces of a fetch
  constexpr int NK = (K_PIECES + THREADS - 1) / THREADS, NV = (V_PIECES + THREADS - 1) / THREADS;  // per thread
  constexpr int K_TILE = PF_BK * KLD, V_TILE = DT * 32 * PF_VLD;              // elements of a parked tile
  constexpr int MERGE_FLOATS = (KP - 1) * RB * (DT * 16 + 2) * DA_WAVE;       // the phases' partial results
  constexpr int TILE_BYTES = NB * (K_TILE + V_TILE) * 2;
  __shared__ __attribute__((aligned(16))) char smem[TILE_BYTES > MERGE_FLOATS * 4 ? TILE_BYTES : MERGE_FLOATS * 4];
  bf16_t (*Ks2)[K_TILE] = (bf16_t (*)[K_TILE])smem;
  bf16_t (*Vs2)[V_TILE] = (bf16_t (*)[V_TILE])(smem + NB * K_TILE * 2);
  __shared__ long long bts[KP == 1 ? PF_BT_MAX : PF_BT_MAX_PHASED];   // a page's place in the cache, in bytes

  // The workgroups with the most keys (the last rows) are launched first, those of every (sequence, head) pair
  // before anybody's second-longest: blockIdx.x, which the dispatcher counts up first, is the pair.  (Counted the
  // other way round, the long workgroups of the later pairs start when the chip is already full of short ones, and
  // the step ends with a few compute units walking their keys alone: at 2 x 4,096 rows and 12 heads the wavefronts
  // resident over the kernel's time averaged 0.9 a SIMD of 2.)
  const int s = seq0 + (int)blockIdx.x / Hq, h = (int)blockIdx.x % Hq;
  const int row0 = q_start[s], T = q_start[s + 1] - row0;
  const int i0 = ((int)gridDim.y - 1 - (int)blockIdx.y) * PF_BQ;
  if (i0 >= T) return;
  const int past = seq_lens[s] - T;
  const int hk = h / (Hq / Hkv);
  const int* bt = block_table + (size_t)s * max_blocks;
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int col = lane % 32, hf = lane / 32;
  const int rbi = wave % RB, kp = wave / RB;       // the wavefront's row block and key phase
  const int wrow = rbi * 32;

  // this lane's query row (as a column of Q^T) and its position
  const int qi = i0 + wrow + col;
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
  const int w_first = past + i0 + wrow;
  const int w_last_row = (i0 + wrow + 31 < T - 1) ? i0 + wrow + 31 : T - 1;
  const bool wave_on = i0 + wrow < T;
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
  float m = -INFINITY, l = 0.f;                 // running maximum (base-2 domain); sum of the weights of this lane half's keys
  const float scale2 = scale * 1.4426950408889634f;

  // The next tile's keys and values are asked for (into registers) before the current tile is
  // multiplied, so their latency hides behind the arithmetic.  Loads are unconditional (a conditional
  // load becomes a branch that serialises them): a key outside b_lo .. b_last reads a key that
  // exists and is replaced by zero.
  // The block table's entries for this workgroup's keys are copied to LDS once: a table entry read
  // from memory in front of every tile would make the tile's loads wait for it, and that wait also
  // drains the loads still in flight for the tiles before.
  const int pg_lo = b_lo >> (31 - __builtin_clz(page)), pg_hi = b_last >> (31 - __builtin_clz(page));
  const long long page_elems = 2LL * Hkv * page * D;
  if (BT_LDS)
    for (int i = t; i <= pg_hi - pg_lo; i += THREADS) bts[i] = bt[pg_lo + i] * page_elems * 2;
  __syncthreads();
  // where a page's keys and values start, in elements from the cache's start
  auto page_at = [&](int key_page) -> long long { return BT_LDS ? bts[key_page - pg_lo] / 2 : bt[key_page] * page_elems; };
  // Two register sets: while a tile is multiplied, the loads of the next two are in flight.
  uint4 rk0[NK], rv0[NV], rk1[NK], rv1[NV];
  const int lg = 31 - __builtin_clz(page);              // page is a power of two (checked on the host)
  const bf16_t* kbase = cache + (long long)hk * page * D;
  const bf16_t* vbase = cache + (long long)(Hkv + hk) * page * D;
  // a tile whose 64 keys all lie in b_lo .. b_last: nothing to clamp, nothing to replace
  // (a fetch covers RT consecutive tiles: key rows kt .. kt + 64 RT - 1; a value piece is 8 keys of
  // one dimension of one tile)
  constexpr int VG = PF_BK / 8, VPT = DT * 32 * VG;       // key groups a tile; value pieces a tile
  // A tile starts at a multiple of 64 keys, a page holds 16, 32 or 64: which page of the tile's pages a thread's
  // piece lies in, and where in that page, never changes.  Both are worked out once; a piece's address is then the
  // page's place (one read of the table in LDS) plus a constant.
  const char* kconst[NK];
  const char* vconst[NV];
  int kpage[NK], vpage[NV];
#pragma unroll
  for (int i = 0; i < NK; ++i) {
    const int c0 = t + i * THREADS, c = c0 < K_PIECES ? c0 : 0;
    const int kr = c / (D / 8), pc = c % (D / 8);
    kpage[i] = kr >> lg;
    kconst[i] = (const char*)(kbase + (kr & (page - 1)) * D + pc * 8);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c0 = t + i * THREADS, c = c0 < V_PIECES ? c0 : 0;
    const int tl = c / VPT, d = (c % VPT) / VG, g = c % VG, k0 = tl * PF_BK + g * 8;
    const int ds = d < D ? d : 0;                        // rows of a padded 32-dimension tile repeat dimension 0
    vpage[i] = k0 >> lg;
    vconst[i] = (const char*)(vbase + ds * page + (k0 & (page - 1)));
  }
  auto page_bytes = [&](int key_page) -> long long { return BT_LDS ? bts[key_page - pg_lo] : bt[key_page] * page_elems * 2; };
  auto fetch_k_fast = [&](uint4* rk, int kt) {
    const int p0 = kt >> lg;
#pragma unroll
    for (int i = 0; i < NK; ++i) rk[i] = *(const uint4*)(kconst[i] + page_bytes(p0 + kpage[i]));
  };
  auto fetch_v_fast = [&](uint4* rv, int kt) {
    const int p0 = kt >> lg;
#pragma unroll
    for (int i = 0; i < NV; ++i) rv[i] = *(const uint4*)(vconst[i] + page_bytes(p0 + vpage[i]));
  };
  auto fetch_fast = [&](uint4* rk, uint4* rv, int kt) {
    fetch_k_fast(rk, kt);
    fetch_v_fast(rv, kt);
  };
  auto fetch_k = [&](uint4* rk, int kt) {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c0 = t + i * THREADS, c = c0 < K_PIECES ? c0 : 0;
      const int kr = c / (D / 8), pc = c % (D / 8), key = kt + kr;
      const bool ok = key >= b_lo && key <= b_last;
      const int ks = ok ? key : b_last;
      rk[i] = *(const uint4*)(kbase + page_at(ks >> lg) + (ks & (page - 1)) * D + pc * 8);
      if (!ok) rk[i] = make_uint4(0, 0, 0, 0);
    }
  };
  auto fetch_v = [&](uint4* rv, int kt) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c0 = t + i * THREADS, c = c0 < V_PIECES ? c0 : 0;
      const int tl = c / VPT, d = (c % VPT) / VG, g = c % VG, key0 = kt + tl * PF_BK + g * 8;   // 8 keys of one dimension
      const bool ok = d < D && key0 + 7 >= b_lo && key0 <= b_last;
      const int ks = ok ? key0 : (b_last / 8) * 8;
      const int ds = d < D ? d : 0;
      uint4 v = *(const uint4*)(vbase + page_at(ks >> lg) + ds * page + (ks & (page - 1)));
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
  auto fetch = [&](uint4* rk, uint4* rv, int kt) {
    fetch_k(rk, kt);
    fetch_v(rv, kt);
  };
  // (one phase: the tile goes to buffer `buf`; KP phases: tile k of the fetch goes to buffer k)
  auto stash_k = [&](const uint4* rk, int buf) {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c = t + i * THREADS, kr = c / (D / 8), pc = c % (D / 8);
      if (K_PIECES % THREADS == 0 || c < K_PIECES) *(uint4*)&Ks2[buf + kr / PF_BK][(kr % PF_BK) * KLD + pc * 8] = rk[i];
    }
  };
  auto stash_v = [&](const uint4* rv, int buf) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = t + i * THREADS, tl = c / VPT, d = (c % VPT) / VG, g = c % VG;
      // Within a block of 16 keys a row keeps them in the order 0-3, 8-11, 4-7, 12-15: the 8 keys a lane
      // multiplies at once (4hf.., 8+4hf.., as the scores' registers hold them) are then 16 consecutive
      // bytes, read in one piece and without bank conflicts.
      if (V_PIECES % THREADS == 0 || c < V_PIECES) {
        bf16_t* vrow = &Vs2[buf + tl][d * PF_VLD + (g / 2) * 16 + (g % 2) * 4];
        *(uint2*)vrow = make_uint2(rv[i].x, rv[i].y);
        *(uint2*)(vrow + 8) = make_uint2(rv[i].z, rv[i].w);
      }
    }
  };
  auto stash = [&](const uint4* rk, const uint4* rv, int buf) {
    stash_k(rk, buf);
    stash_v(rv, buf);
  };
  const int kt0 = (b_lo / (RT * PF_BK)) * (RT * PF_BK);
  // The scores of one tile, out of LDS buffer `buf`: S^T = K . Q^T.
  auto scores = [&](int buf, floatx16 (&sc)[2]) {
    const bf16_t* Ks = Ks2[buf];
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
  };
  // Mask, running maximum, weights, and the weighted sum of the tile's values out of LDS buffer `buf`.
  // WHOLE: every row of the wavefront sees all of the tile's keys, known when compiled (no mask, no branch).
  auto weigh = [&](int kt, int buf, floatx16 (&sc)[2], auto wholec) {
    constexpr bool WHOLE = decltype(wholec)::value;
    const bf16_t* Vs = Vs2[buf];
    {
      // Mask, running maximum and weights.  The maximum is kept in the base-2 domain
      // (s * scale * log2 e, scale > 0), so that a weight costs one multiply-add and one hardware
      // exp2.  A tile that every row of the wavefront sees whole needs no mask at all; elsewhere a key
      // outside q_lo .. pq gets -inf added (0 otherwise), computed from the sign of
      // min(pq - key, key - q_lo) without a comparison: scores are finite, keys that do not exist
      // were loaded as zeros.
      const bool whole = WHOLE || (kt + PF_BK - 1 <= w_first && (window <= 0 || kt >= w_last - window + 1));
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
      tmax = half_max(tmax) * scale2;                  // over both halves of the wavefront: all 64 keys of the row
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
      l = l * alpha + tsum;                            // this half's keys only: the halves' sums meet at the end
      m = m_new;
      // (skipping this when no row's maximum rose was measured: no gain, some row of 32 mostly has a new one)
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] *= alpha;
      // O^T += V^T . P^T ; the lane's 8 keys of a 16-key block are 4hf..4hf+3 and 8+4hf..8+4hf+3, which
      // lie side by side in the parked tile
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
            const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, *(const uint4*)&Vs[(i * 32 + col) * PF_VLD + ks * 32 + kb * 16 + 8 * hf]);
            acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[ks][kb], acc_o[i], 0, 0, 0);
          }
    }
  };
  // the products of one tile, out of LDS buffer `buf`
  auto tile = [&](int kt, int buf) {
    if (wave_on && kt <= w_last && kt + PF_BK - 1 >= w_lo) {
      floatx16 sc[2];
      scores(buf, sc);
      weigh(kt, buf, sc, std::false_type{});
    }
  };

  // Steady state, two tiles a round, without a branch around the loads: the compiler then counts the
  // loads in flight exactly and a tile waits for its own registers only.  It lasts while the tile
  // asked for (two ahead) lies whole inside the workgroup's keys; the last tiles run through the
  // same steps with conditions and the clamping loads.  One barrier a tile: the buffer written now
  // was last read two tiles ago, before the previous barrier.
  if constexpr (KP == 1) {
  int kt = kt0;
  // Where the keys start at a tile's edge (no window, or one that happens to) and the steady state runs
  // at least once, its first two tiles are asked for the way it asks for all others: the loop is then
  // entered with the same loads in flight, in the same order, as it is re-entered, and the compiler counts
  // exactly how many may stay in flight at each wait.  (Entered after the clamping loads it waited for all
  // of them, and every second tile's keys had one tile's time to arrive instead of two.)  Elsewhere the
  // loop below, which takes any tile, does all of them.
  if (b_lo == kt0 && kt0 + 4 * PF_BK - 1 <= b_last) {
    fetch_fast(rk0, rv0, kt0);
    fetch_fast(rk1, rv1, kt0 + PF_BK);
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
  } else {
    fetch(rk0, rv0, kt0);
    if (kt0 + PF_BK <= b_last) fetch(rk1, rv1, kt0 + PF_BK);
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
  } else {
    // Key phases: a round parks KP tiles (one register set: the next round's loads fly while this
    // round's tiles are multiplied), each wavefront multiplies the tile of its phase.  Two barriers a
    // round: the tiles are parked before anyone reads them and read before they are replaced.
    if (b_lo == kt0 && kt0 + KP * PF_BK - 1 <= b_last) fetch_fast(rk0, rv0, kt0);     // (a first round that is whole: no clamping)
    else fetch(rk0, rv0, kt0);
    for (int kt = kt0; kt <= b_last; kt += KP * PF_BK) {
      stash(rk0, rv0, 0);
      lds_barrier();
      const int nx = kt + KP * PF_BK;
      if (nx + KP * PF_BK - 1 <= b_last) fetch_fast(rk0, rv0, nx);     // (nx >= b_lo: only the first round starts below it)
      else if (nx <= b_last) fetch(rk0, rv0, nx);
      tile(kt + kp * PF_BK, kp);
      lds_barrier();
    }
    // the phases' partial results, merged by phase 0 in the order of the phases
    l += __shfl_xor(l, 32, DA_WAVE);                    // (both halves had the same maximum all along)
    float* mg = (float*)smem;
    constexpr int PER = DT * 16 + 2;
    if (kp > 0) {
      float* mine = mg + (size_t)((kp - 1) * RB + rbi) * PER * DA_WAVE + lane;
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[(i * 16 + r) * DA_WAVE] = acc_o[i][r];
      mine[(DT * 16) * DA_WAVE] = m;
      mine[(DT * 16 + 1) * DA_WAVE] = l;
    }
    lds_barrier();
    if (kp > 0) return;
#pragma unroll
    for (int k = 1; k < KP; ++k) {
      const float* theirs = mg + (size_t)((k - 1) * RB + rbi) * PER * DA_WAVE + lane;
      const float mk = theirs[(DT * 16) * DA_WAVE], lk = theirs[(DT * 16 + 1) * DA_WAVE];
      const float m_new = fmaxf(m, mk);
      const float m_use = m_new != -INFINITY ? m_new : 0.f;
      const float a0 = __builtin_amdgcn_exp2f(m - m_use), a1 = __builtin_amdgcn_exp2f(mk - m_use);
      l = l * a0 + lk * a1;
      m = m_new;
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = acc_o[i][r] * a0 + theirs[(i * 16 + r) * DA_WAVE] * a1;
    }
  }

  if constexpr (KP == 1) l += __shfl_xor(l, 32, DA_WAVE);   // (both halves had the same maximum all along)
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
                               void* out, int out_ld, int form, void* stream) {
  DA_REQUIRE(n_seqs >= 0 && Hq > 0 && Hkv > 0 && page > 0 && max_query_len >= 0, "attn_prefill: bad sizes");
  DA_REQUIRE(Hq % Hkv == 0, "attn_prefill: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(D % 16 == 0 && D >= 16 && D <= 256, "attn_prefill: head size %d is not a multiple of 16 up to 256", D);
  DA_REQUIRE(page >= 8 && (page & (page - 1)) == 0 && PF_BK % page == 0, "attn_prefill: page size %d must be 8, 16, 32 or 64", page);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * D && q_ld % 8 == 0 && out_ld % 4 == 0, "attn_prefill: row lengths");
  DA_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)cache % 16 == 0) && ((uintptr_t)out % 8 == 0),
             "attn_prefill: operands must be 16-byte aligned");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_prefill: bad window or block table");
  DA_REQUIRE(scale > 0.f, "attn_prefill: the score scale must be positive, found %g", (double)scale);
  DA_REQUIRE((long)n_seqs * Hq < (1L << 31) && max_query_len <= 65535 * 32, "attn_prefill: too many sequences, heads or rows for one launch");
  if (n_seqs == 0 || max_query_len == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  // The workgroup's form, row blocks x key phases.  Short portions (after a long past, beside decoded
  // tokens) have few rows to a sequence and head: 1 x 4 up to 32 rows, 2 x 2 up to 64, so that all four
  // wavefronts work and share out the keys.  Longer ones take 128 rows a workgroup (smaller row blocks
  // read the keys more often, and that traffic binds), and 4 x 2, eight wavefronts, while there is no
  // more than one workgroup a compute unit; else 4 x 1.  Measured on MI355X, head size 64, microseconds
  // 4x1 / 4x2 / 2x2 / 1x4: 2 x 1,024 rows, 12 heads 23.3 / 19.3 / 23.4 / 34.6; 2,048 rows 40.0 / 31.8 /
  // 38.9 / 51.7; 8 x 512 rows 19.3 / 23.3 / 26.2 / 42.5; 4 x 64 rows after 900 keys 22.8 / 17.8 / 17.8 /
  // 16.3; 16 x 2 rows after 1,000 keys 22.8 / 18.5 / 18.3 / 18.0.  With the longest workgroups of every pair launched
  // first, 4x1 / 4x2: 2 x 1,024 rows, 12 heads 23.2 / 20.0, 25 heads 26.0 / 25.5; 8 x 1,024 rows, 12 heads 35.5 / 39.9;
  // 2 x 4,096 rows 93.6 / 108.5 (551 TFLOP/s; 157.6 before); 8,192 rows 165.5 / 190.2; 4 x 512 rows after 512 keys,
  // 16 heads 22.5 / 19.7.  Workgroups of 256 rows (8 x 1) were behind 4 x 1 at every one of these.  A loop that multiplies
  // the scores of tile j + 1 while tile j is weighed (keys parked one tile ahead of values) gave the same bits and
  // -8 % to +12 % of 4 x 1's time depending on the shape: with two wavefronts a SIMD the matrix cores already run under
  // the other wavefront's softmax; it is not kept.  Four key phases (2 x 4, 4 x 4) were behind 4 x 2 at every shape (2 x
  // 1,024 rows, 12 heads: 20.5 and 22.3 against 18.3 us): a round's two barriers and the merge cost more than they share out.
  // Forms with phases need their tiles in LDS at once: head sizes up to 64 (4 x 2, 1 x 4) or 128 (2 x 2).  The
  // choice reads the step's shape only.
  // form: 0 leaves the choice to this rule; 41, 42, 22 or 14 fixes it
  const long per128 = (long)da_ceil_div(max_query_len, 128) * Hq * n_seqs;
  const int chosen = form ? form
                     : (D <= 64 && max_query_len <= 32) ? 14
                     : (D <= 128 && max_query_len <= 64) ? 22
                     : (D <= 64 && per128 <= PF_PHASED_MAX_WORKGROUPS) ? 42 : 41;
  DA_REQUIRE(chosen == 41 || (chosen == 22 && D <= 128) || ((chosen == 42 || chosen == 14) && D <= 64),
             "attn_prefill: form %d with a head size of %d (41 for any; 22 up to 128; 42 and 14 up to 64)", chosen, D);
  // every key a workgroup can see lies within max_blocks pages
  const bool bt_lds = max_blocks <= (chosen == 41 ? PF_BT_MAX : PF_BT_MAX_PHASED);
#define LAUNCH2(N, RB, KP, L)                                                                                  \
  hipLaunchKernelGGL((attn_prefill_kernel<N, RB, KP, L>), dim3(Hq * n_seqs, da_ceil_div(max_query_len, 32 * RB)), \
                     dim3(RB * KP * DA_WAVE), 0, st, (const bf16_t*)q, q_ld, (const bf16_t*)cache, block_table, \
                     max_blocks, q_start, seq_lens, seq0, Hq, Hkv, page, scale, window, (bf16_t*)out, out_ld)
#define LAUNCH3(N, RB, KP)                \
  do {                                    \
    if (bt_lds) LAUNCH2(N, RB, KP, true); \
    else LAUNCH2(N, RB, KP, false);       \
  } while (0)
#define LAUNCH_SMALL(N)                     \
  case N:                                   \
    if (chosen == 14) LAUNCH3(N, 1, 4);     \
    else if (chosen == 22) LAUNCH3(N, 2, 2); \
    else if (chosen == 42) LAUNCH3(N, 4, 2); \
    else LAUNCH3(N, 4, 1);                  \
    break;
#define LAUNCH_MID(N)                       \
  case N:                                   \
    if (chosen == 22) LAUNCH3(N, 2, 2);     \
    else LAUNCH3(N, 4, 1);                  \
    break;
#define LAUNCH(N)                           \
  case N:                                   \
    LAUNCH3(N, 4, 1);                       \
    break;
  switch (D / 16) {
    LAUNCH_SMALL(1) LAUNCH_SMALL(2) LAUNCH_SMALL(3) LAUNCH_SMALL(4) LAUNCH_MID(5) LAUNCH_MID(6) LAUNCH_MID(7) LAUNCH_MID(8)
    LAUNCH(9) LAUNCH(10) LAUNCH(11) LAUNCH(12) LAUNCH(13) LAUNCH(14) LAUNCH(15) LAUNCH(16)
  }
#undef LAUNCH
#undef LAUNCH_MID
#undef LAUNCH_SMALL
#undef LAUNCH3
#undef LAUNCH2
  DA_CHECK_LAUNCH("attn_prefill");
  return 0;
}
