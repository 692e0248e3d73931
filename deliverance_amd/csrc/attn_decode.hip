// Paged attention for decode rows in bfloat16: one query row per sequence.
//
// One workgroup of 8 wavefronts per (sequence, query head).  The keys lo..p of the sequence
// are walked in aligned chunks of 64; wavefront v takes chunks v, v+8, ... (two each at a
// context of 1,024).  All loads of a phase are issued before any is used, so a chunk costs two
// memory round trips.
//   scores : CPR lanes share a key, each holding a 16-byte piece of the key row and the matching
//            piece of q in registers; their partial dot products are added by lane exchange.
//            One load instruction so covers 64 / CPR whole key rows that lie next to each other.
//   softmax: every lane ends up with one key's score; running maximum and sum per wavefront
//            (the recurrence of native/src/main/resources/decode_paged_attention_f32.wgsl:31-65).
//   values : values are stored dimension-major, so lane d reads 8 consecutive keys of its own
//            dimension in 16 bytes and keeps one accumulator; no exchange between lanes.
// The wavefronts' partial results are merged in LDS in a fixed order.  Every sum's order
// depends on p and lo only, never on the batch.
//
// Formulas: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:504-532;
// tensor/src/main/java/io/teknek/deliverance/tensor/operations/TensorOperations.java:240-272.
#include "common.h"

#define DEC_MAX_D 256

// e^x by the hardware's exp2 (two instructions; the library's expf is a dozen, and the merge of 16 wavefronts'
// partial results takes 16 of them on the one wavefront that everything waits for)
__device__ __forceinline__ float dec_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// Long contexts with few (sequence, head) pairs: the keys are also split over workgroups.  Workgroup
// (pair, j) takes the keys j * span .. (j + 1) * span - 1 (span a multiple of 64) and leaves its
// partial result (the weighted sum before the division, the maximum, the sum of weights: D + 2
// floats) in a scratch buffer; a second kernel merges a pair's partial results in ascending order
// of j.  The split depends on the step's shape only (pairs, widest block table), never on the
// sequences' lengths, so a recorded graph can hold it.
//
// CPR: 16-byte pieces per key row, rounded up to a power of two (2..32)
template <int CPR, int DEC_WAVES, bool SPLIT>
// (registers are held to 128 for head sizes up to 64, so that two workgroups share a compute unit)
__global__ void __launch_bounds__(DEC_WAVES * DA_WAVE, (CPR <= 8 || DEC_WAVES == 16) ? 4 : 2)
attn_decode_kernel(const bf16_t* __restrict__ q, int q_ld, const bf16_t* __restrict__ cache,
                   const int* __restrict__ block_table, int max_blocks,
                   const int* __restrict__ seq_lens, int Hq, int Hkv, int D, int page, float scale,
                   int window, bf16_t* __restrict__ out, int out_ld, int span, float* __restrict__ partial) {
  constexpr int G = DA_WAVE / CPR;            // keys scored side by side
  constexpr int DPL = CPR <= 8 ? 1 : CPR / 8; // value dimensions per lane: D <= 8 * CPR <= 64 * DPL
  __shared__ __attribute__((aligned(16))) float ps[DEC_WAVES][DA_WAVE];
  __shared__ float part_acc[DEC_WAVES][DPL * DA_WAVE];
  __shared__ float part_m[DEC_WAVES], part_l[DEC_WAVES];

  const int s = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const int hk = h / (Hq / Hkv);
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int* bt = block_table + (size_t)s * max_blocks;
  // addressing by shifts: the page size is a power of two (checked on the host)
  const int lg = 31 - __builtin_clz(page), pmask = page - 1;
  const long long page_elems = 2LL * Hkv * page * D;
  const bf16_t* kbase = cache + (long long)hk * page * D;
  const bf16_t* vbase = cache + (long long)(Hkv + hk) * page * D;
  const int piece = lane % CPR, sub = lane / CPR;
  const bool piece_ok = piece * 8 < D;

  // Asked for before the sequence's length is known, so that they travel beside it: the query (as
  // raw bits; converted where it is used) and the block-table entries of the chunk this wavefront
  // starts with when nothing is cut off by a window (keys wave*64 ..).  Entries past the
  // sequence's pages are read (the table has max_blocks of them) and never used.
  const uint4 qraw = *(const uint4*)(q + (size_t)s * q_ld + h * D + (piece_ok ? piece * 8 : 0));
  const int split0 = SPLIT ? (int)blockIdx.y * span : 0;          // the first key of this workgroup's share
  const int c0_guess = split0 + wave * DA_WAVE;
  // (head sizes above 128 have no registers to spare for them and read the table chunk by chunk)
  constexpr bool EARLY_BT = CPR <= 16;
  int btk0[EARLY_BT ? CPR : 1], btv0[EARLY_BT ? 8 : 1];
  if (EARLY_BT) {
#pragma unroll
    for (int i = 0; i < (EARLY_BT ? CPR : 1); ++i) {
      const int pg = (c0_guess + i * G + sub) >> lg;
      btk0[i] = bt[pg < max_blocks ? pg : max_blocks - 1];
    }
#pragma unroll
    for (int g = 0; g < (EARLY_BT ? 8 : 1); ++g) {
      const int pg = (c0_guess + g * 8) >> lg;
      btv0[g] = bt[pg < max_blocks ? pg : max_blocks - 1];
    }
  }
  // the row's position is seq_lens[s] - 1; it sees the keys lo..p (of which this workgroup takes its share)
  const int p_row = seq_lens[s] - 1;
  const int lo_row = (window > 0 && p_row - window + 1 > 0) ? p_row - window + 1 : 0;
  const int p = SPLIT ? (p_row < split0 + span - 1 ? p_row : split0 + span - 1) : p_row;
  const int lo = SPLIT ? (lo_row > split0 ? lo_row : split0) : lo_row;

  float acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int c0 = (lo / DA_WAVE) * DA_WAVE + wave * DA_WAVE; c0 <= p; c0 += DEC_WAVES * DA_WAVE) {
    // ---- all loads of the chunk first: the key pieces of the score phase and the value groups
    // of the weighted sum (both need only the block table), then the arithmetic
    float mine = -INFINITY;      // one key's score per lane, once the loop is done
    uint4 kv[CPR];
    const int first = c0 > lo ? c0 : lo;                 // valid keys of the chunk: first..last
    const int last = c0 + DA_WAVE - 1 < p ? c0 + DA_WAVE - 1 : p;
    // the pages of the chunk's keys and value groups: those asked for at the start, or read now
    int btk[CPR], btv[8], bt_safe;
    if (EARLY_BT && c0 == c0_guess && first == c0) {     // the same for the whole wavefront
#pragma unroll
      for (int i = 0; i < CPR; ++i) btk[i] = btk0[EARLY_BT ? i : 0];
#pragma unroll
      for (int g = 0; g < 8; ++g) btv[g] = btv0[EARLY_BT ? g : 0];
      bt_safe = __builtin_amdgcn_readfirstlane(btk0[0]); // lane 0 holds the page of key c0
    } else if (CPR == 32) {
      // Two keys a load, both in one page (a page has 8 rows at least), and the chunk is the same for
      // the whole wavefront: the table entries are read by the scalar unit and take no vector registers,
      // which this head size has none to spare of.
      const int c0u = __builtin_amdgcn_readfirstlane(c0), fu = __builtin_amdgcn_readfirstlane(first),
                lu = __builtin_amdgcn_readfirstlane(last);
      bt_safe = __builtin_amdgcn_readfirstlane(bt[fu >> lg]);
#pragma unroll
      for (int i = 0; i < CPR; ++i) {
        const int k0 = c0u + i * G;                      // the load's first key; G = 2
        btk[i] = __builtin_amdgcn_readfirstlane(bt[((k0 + G - 1 >= fu && k0 <= lu) ? k0 : fu) >> lg]);
      }
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        const int g0 = c0u + g * 8;
        btv[g] = __builtin_amdgcn_readfirstlane(bt[((g0 + 7 >= fu && g0 <= lu) ? g0 : fu) >> lg]);
      }
    } else {
      bt_safe = bt[first >> lg];
#pragma unroll
      for (int i = 0; i < CPR; ++i) {
        const int key = c0 + i * G + sub;
        btk[i] = bt[((key >= first && key <= last) ? key : first) >> lg];
      }
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        const int g0 = c0 + g * 8;
        btv[g] = bt[((g0 + 7 >= first && g0 <= last) ? g0 : first) >> lg];
      }
    }
    // a key that is not seen reads `first` instead, a row that surely exists
#pragma unroll
    for (int i = 0; i < CPR; ++i) {
      const int key = c0 + i * G + sub;
      const bool valid = key >= lo && key <= p;
      // (CPR 32: btk[i] is the pair's page, or the page of `first` if neither key is seen, the same for every
      // lane: the page's address stays with the scalar unit; a lane whose own key is not seen reads some row of it)
      const long long pg = CPR == 32 ? btk[i] : (valid ? btk[i] : bt_safe);
      const int kk = valid ? key : first;
      kv[i] = *(const uint4*)(kbase + pg * page_elems + (kk & pmask) * D + (piece_ok ? piece * 8 : 0));
    }
    // the chunk's 8 groups of 8 keys (a group never crosses a page) of this lane's first dimension;
    // groups with no seen key read the group of `first` instead and are dropped
    // (head sizes above 128 hold 128 registers of keys at this point: their values are asked for once the
    // scores are done, all dimensions at once)
    constexpr bool EARLY_V = CPR <= 16;
    uint4 vv0[8];
    if (EARLY_V) {
      const int d = lane < D ? lane : 0;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        const int g0 = c0 + g * 8;
        const bool any = g0 + 7 >= first && g0 <= last;
        const int gs = any ? g0 : (first / 8) * 8;
        const long long pg = any ? btv[g] : bt_safe;
        vv0[g] = *(const uint4*)(vbase + pg * page_elems + d * page + (gs & pmask));
      }
    }
    // nothing moves across this line: the compiler would otherwise push the value loads down behind
    // the scores to save registers, and a chunk would cost a third memory round trip
    __builtin_amdgcn_sched_barrier(0);
    float qf[8];
    {
      const uint32_t u[4] = {qraw.x, qraw.y, qraw.z, qraw.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qf[2 * e] = piece_ok ? __uint_as_float(u[e] << 16) * scale : 0.f;
        qf[2 * e + 1] = piece_ok ? __uint_as_float(u[e] & 0xffff0000u) * scale : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < CPR; ++i) {
      const int key = c0 + i * G + sub;
      const bool valid = key >= lo && key <= p;
      const uint32_t u[4] = {kv[i].x, kv[i].y, kv[i].z, kv[i].w};
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        dot = fmaf(qf[2 * e], __uint_as_float(u[e] << 16), dot);
        dot = fmaf(qf[2 * e + 1], __uint_as_float(u[e] & 0xffff0000u), dot);
      }
      dot = group_sum<CPR>(dot);
      // all CPR lanes of the group now hold the score; the lane whose piece number is i keeps it
      if (piece == i) mine = valid ? dot : -INFINITY;
    }
    const int kidx = piece * G + sub;                 // which key of the chunk this lane kept
    const int key = c0 + kidx;
    const bool valid = key >= lo && key <= p;
    const float m_new = fmaxf(m, wave_max(mine));
    const float e = valid ? dec_exp(mine - m_new) : 0.f;
    const float alpha = dec_exp(m - m_new);
    l = l * alpha + wave_sum(e);
    m = m_new;
    ps[wave][kidx] = e;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");   // LDS only: the value loads stay in flight
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    // ---- values: lane owns dimensions lane, lane + 64, ...; what was not asked for ahead of the scores is
    // asked for now, every dimension's loads before any is used
    uint4 vall[DPL][8];
    if (!EARLY_V) __builtin_amdgcn_sched_barrier(0);    // (not moved up among the scores: the keys' registers are free only now)
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      if (EARLY_V && i == 0) {
#pragma unroll
        for (int g = 0; g < 8; ++g) vall[0][g] = vv0[g];
      } else {
        const int di = lane + i * DA_WAVE, d = di < D ? di : 0;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          const int g0 = c0 + g * 8;
          const bool any = g0 + 7 >= first && g0 <= last;
          const int gs = any ? g0 : (first / 8) * 8;
          const long long pg = any ? btv[g] : bt_safe;
          vall[i][g] = *(const uint4*)(vbase + pg * page_elems + d * page + (gs & pmask));
        }
      }
    }
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + i * DA_WAVE;
      if (DPL > 1 && d >= D) break;
      float a = acc[i] * alpha;
      const uint4* vv = vall[i];
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        // Rows outside first..last were never written (or belong to someone else) and may hold anything:
        // their bits are cleared.  The seen rows of a group are g0+lo8 .. g0+hi8; the masks are the same
        // for every lane, so the scalar unit builds them.
        const int g0 = c0 + g * 8;
        const int lo8 = first - g0 > 0 ? first - g0 : 0, hi8 = last - g0 < 7 ? last - g0 : 7;
        uint32_t msk[4];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2)
          msk[e2] = ((2 * e2 >= lo8 && 2 * e2 <= hi8) ? 0x0000ffffu : 0u) |
                    ((2 * e2 + 1 >= lo8 && 2 * e2 + 1 <= hi8) ? 0xffff0000u : 0u);
        const uint32_t u[4] = {vv[g].x & msk[0], vv[g].y & msk[1], vv[g].z & msk[2], vv[g].w & msk[3]};
        const float4 w0 = *(const float4*)&ps[wave][g * 8];
        const float4 w1 = *(const float4*)&ps[wave][g * 8 + 4];
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          a = fmaf(w[2 * e2], __uint_as_float(u[e2] << 16), a);
          a = fmaf(w[2 * e2 + 1], __uint_as_float(u[e2] & 0xffff0000u), a);
        }
      }
      acc[i] = a;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");   // LDS only: the value loads stay in flight
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = lane + i * DA_WAVE;
    if (d < D) part_acc[wave][d] = acc[i];
  }
  if (lane == 0) { part_m[wave] = m; part_l[wave] = l; }
  __syncthreads();
  // merge the wavefronts' partial softmaxes in a fixed order
  float mm = part_m[0];
#pragma unroll
  for (int w2 = 1; w2 < DEC_WAVES; ++w2) mm = fmaxf(mm, part_m[w2]);
  float ll = 0.f;
  float f[DEC_WAVES];
#pragma unroll
  for (int w2 = 0; w2 < DEC_WAVES; ++w2) {
    f[w2] = part_m[w2] == -INFINITY ? 0.f : dec_exp(part_m[w2] - mm);
    ll += part_l[w2] * f[w2];
  }
  if (SPLIT) {
    // the share's result before the division, its maximum and its sum of weights
    float* mine = partial + ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * (D + 2);
    for (int d = t; d < D; d += DEC_WAVES * DA_WAVE) {
      float o = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < DEC_WAVES; ++w2) o += part_acc[w2][d] * f[w2];
      mine[d] = o;
    }
    if (t == 0) { mine[D] = mm; mine[D + 1] = ll; }
    return;
  }
  const float inv = ll > 0.f ? 1.0f / ll : 0.f;     // a sequence of length 0 (padding) gives zeros
  for (int d = t; d < D; d += DEC_WAVES * DA_WAVE) {
    float o = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < DEC_WAVES; ++w2) o += part_acc[w2][d] * f[w2];
    out[(size_t)s * out_ld + h * D + d] = f32_to_bf16(o * inv);
  }
}

// The partial results of a (sequence, head) pair, merged in ascending order of the shares.
__global__ void __launch_bounds__(256)
attn_decode_merge_kernel(const float* __restrict__ partial, int n_splits, int Hq, int D,
                         bf16_t* __restrict__ out, int out_ld) {
  const int s = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const float* mine = partial + (size_t)blockIdx.x * n_splits * (D + 2);
  float mm = -INFINITY;
  for (int j = 0; j < n_splits; ++j) mm = fmaxf(mm, mine[(size_t)j * (D + 2) + D]);
  float ll = 0.f;
  for (int j = 0; j < n_splits; ++j) {
    const float mj = mine[(size_t)j * (D + 2) + D];
    ll += mine[(size_t)j * (D + 2) + D + 1] * (mj == -INFINITY ? 0.f : dec_exp(mj - mm));
  }
  const float inv = ll > 0.f ? 1.0f / ll : 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float o = 0.f;
    for (int j = 0; j < n_splits; ++j) {
      const float mj = mine[(size_t)j * (D + 2) + D];
      o += mine[(size_t)j * (D + 2) + d] * (mj == -INFINITY ? 0.f : dec_exp(mj - mm));
    }
    out[(size_t)s * out_ld + h * D + d] = f32_to_bf16(o * inv);
  }
}

static int decode_checks(const void* q, int q_ld, const void* cache, int max_blocks, int S, int Hq, int Hkv, int D,
                         int page, int window, int out_ld) {
  DA_REQUIRE(S >= 0 && Hq > 0 && Hkv > 0 && page > 0, "attn_decode: bad sizes");
  DA_REQUIRE(Hq % Hkv == 0, "attn_decode: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(D % 16 == 0 && D >= 16 && D <= DEC_MAX_D, "attn_decode: head size %d is not a multiple of 16 up to %d", D, DEC_MAX_D);
  DA_REQUIRE(page % 8 == 0 && DA_WAVE % page == 0, "attn_decode: page size %d must be 8, 16, 32 or 64", page);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * D, "attn_decode: row lengths too small");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_decode: bad window or block table");
  DA_REQUIRE((uintptr_t)cache % 16 == 0 && (uintptr_t)q % 16 == 0 && q_ld % 8 == 0,
             "attn_decode: q and the cache must be 16-byte aligned");
  return 0;
}

// n_splits == 1: one workgroup a (sequence, head) pair, no scratch.  n_splits > 1: the keys of a pair
// go to n_splits workgroups of `span` keys each, partial results through `partial`
// (S * Hq * n_splits * (D + 2) floats), then the merge kernel.
static int decode_launch(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks,
                         const int* seq_lens, int S, int Hq, int Hkv, int D, int page, float scale, int window,
                         void* out, int out_ld, int n_splits, int span, float* partial, hipStream_t st) {
  const int pieces = D / 8;
  // 8 wavefronts; 16 where the workgroups are no more than the compute units (a context above 512 is then
  // still one chunk a wavefront, and the larger workgroup's start is paid once per compute unit)
  const bool wide = (long)S * Hq * n_splits <= 256 && pieces <= 8;     // larger heads need the registers of 8 wavefronts
  dim3 grid(S * Hq, n_splits);
#define LAUNCH3(C, W, SP)                                                                                   \
  hipLaunchKernelGGL((attn_decode_kernel<C, W, SP>), grid, dim3(W * DA_WAVE), 0, st, (const bf16_t*)q, q_ld, \
                     (const bf16_t*)cache, block_table, max_blocks, seq_lens, Hq, Hkv, D, page, scale, window, \
                     (bf16_t*)out, out_ld, span, partial)
#define LAUNCH2(C, W) do { if (n_splits > 1) LAUNCH3(C, W, true); else LAUNCH3(C, W, false); } while (0)
#define LAUNCH(C) do { if (wide) LAUNCH2(C, 16); else LAUNCH2(C, 8); } while (0)
  if (pieces <= 2) LAUNCH(2);
  else if (pieces <= 4) LAUNCH(4);
  else if (pieces <= 8) LAUNCH(8);
  else if (pieces <= 16) LAUNCH2(16, 8);
  else LAUNCH2(32, 8);
#undef LAUNCH
#undef LAUNCH2
#undef LAUNCH3
  if (n_splits > 1)
    hipLaunchKernelGGL(attn_decode_merge_kernel, dim3(S * Hq), dim3(D <= 64 ? 64 : (D <= 128 ? 128 : 256)), 0, st,
                       partial, n_splits, Hq, D, (bf16_t*)out, out_ld);
  return 0;
}

extern "C" int da_attn_decode(const void* q, int q_ld, const void* cache, const int* block_table,
                              int max_blocks, const int* seq_lens, int S, int Hq, int Hkv, int D, int page,
                              float scale, int window, void* out, int out_ld, void* stream) {
  if (decode_checks(q, q_ld, cache, max_blocks, S, Hq, Hkv, D, page, window, out_ld)) return 1;
  if (S == 0) return 0;
  decode_launch(q, q_ld, cache, block_table, max_blocks, seq_lens, S, Hq, Hkv, D, page, scale, window, out, out_ld,
                1, 0, nullptr, (hipStream_t)stream);
  DA_CHECK_LAUNCH("attn_decode");
  return 0;
}

// The keys of every (sequence, head) pair split over n_splits workgroups; `workspace` holds the
// partial results (da_attn_decode_split_bytes of it, 16-byte aligned).
extern "C" long da_attn_decode_split_bytes(int S, int Hq, int D, int n_splits) {
  return (long)S * Hq * n_splits * (D + 2) * (long)sizeof(float);
}

static int split_checks(int max_blocks, int page, int n_splits, int* span) {
  DA_REQUIRE(n_splits >= 2 && n_splits <= 64, "attn_decode_split: %d shares (2 to 64 are taken)", n_splits);
  const long keys = (long)max_blocks * page;
  *span = (int)(((keys + n_splits - 1) / n_splits + DA_WAVE - 1) / DA_WAVE * DA_WAVE);
  return 0;
}

extern "C" int da_attn_decode_split(const void* q, int q_ld, const void* cache, const int* block_table,
                                    int max_blocks, const int* seq_lens, int S, int Hq, int Hkv, int D, int page,
                                    float scale, int window, void* out, int out_ld, int n_splits, void* workspace,
                                    long workspace_bytes, void* stream) {
  if (decode_checks(q, q_ld, cache, max_blocks, S, Hq, Hkv, D, page, window, out_ld)) return 1;
  int span = 0;
  if (split_checks(max_blocks, page, n_splits, &span)) return 1;
  DA_REQUIRE(workspace && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= da_attn_decode_split_bytes(S, Hq, D, n_splits),
             "attn_decode_split: the workspace holds %ld bytes, %ld are needed", workspace_bytes,
             da_attn_decode_split_bytes(S, Hq, D, n_splits));
  if (S == 0) return 0;
  decode_launch(q, q_ld, cache, block_table, max_blocks, seq_lens, S, Hq, Hkv, D, page, scale, window, out, out_ld,
                n_splits, span, (float*)workspace, (hipStream_t)stream);
  DA_CHECK_LAUNCH("attn_decode_split");
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The same without a workspace argument and without any allocation (see no_alloc.h).
// ---------------------------------------------------------------------------------------------
#include "no_alloc.h"
#include <mutex>

static __device__ __align__(256) unsigned char scratch[DA_DECODE_STATIC_SCRATCH_BYTES];

#define DA_MAX_DEVICES 64
static void* g_scratch_of_device[DA_MAX_DEVICES];      // the array's address on each GPU, asked for once
static std::mutex g_scratch_mutex;

// The address of `scratch` on the current device.  In host code the array's name is only a handle
// for the runtime; the memory's address differs from GPU to GPU and comes from hipGetSymbolAddress.
static int static_scratch(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  DA_REQUIRE(e == hipSuccess && dev >= 0 && dev < DA_MAX_DEVICES, "attn_decode_split_static: no current device (%s)",
             hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    DA_REQUIRE(e == hipSuccess && p, "attn_decode_split_static: the scratch buffer's address is not known (%s)",
               hipGetErrorString(e));
    g_scratch_of_device[dev] = p;
  }
  *ptr = (float*)g_scratch_of_device[dev];
  return 0;
}

extern "C" int da_attn_decode_split_static(const void* q, int q_ld, const void* cache, const int* block_table,
                                           int max_blocks, const int* seq_lens, int S, int Hq, int Hkv, int D,
                                           int page, float scale, int window, void* out, int out_ld, int n_splits,
                                           void* stream) {
  if (decode_checks(q, q_ld, cache, max_blocks, S, Hq, Hkv, D, page, window, out_ld)) return 1;
  int span = 0;
  if (split_checks(max_blocks, page, n_splits, &span)) return 1;
  const long need = da_attn_decode_split_bytes(S, Hq, D, n_splits);
  DA_REQUIRE(need <= (long)DA_DECODE_STATIC_SCRATCH_BYTES,
             "attn_decode_split_static: %d sequences x %d heads x %d shares of head size %d need %ld bytes of scratch, "
             "the library holds %ld", S, Hq, n_splits, D, need, (long)DA_DECODE_STATIC_SCRATCH_BYTES);
  if (S == 0) return 0;
  float* partial = nullptr;
  if (static_scratch(&partial)) return 1;
  decode_launch(q, q_ld, cache, block_table, max_blocks, seq_lens, S, Hq, Hkv, D, page, scale, window, out, out_ld,
                n_splits, span, partial, (hipStream_t)stream);
  DA_CHECK_LAUNCH("attn_decode_split_static");
  return 0;
}
