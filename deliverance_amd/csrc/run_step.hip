// One step of a model of standard parts, launch after launch, from C++ (see run_step.h).
#include "run_step.h"
#include "common.h"

extern "C" {
int da_embed(const int* tokens, const int* positions, const void* wte, int wte_dtype, const void* wpe, int wpe_dtype,
             float* x, int N, int E, float scale, void* stream);
int da_layernorm(const float* x, const int* rows, const void* w, int w_dtype, const void* b, int b_dtype, float eps,
                 void* y, int y_dtype, int R, int E, void* stream);
int da_gemm_bf16(const void* a, int lda, const void* w, int ldw, const void* bias, int bias_dtype, int act, int accumulate,
                 void* out, int out_dtype, int ldo, int M, int N, int K, void* kv_cache, const int* slot_map, int q_cols,
                 int kv_cols, int Hkv, int D, int page, void* stream);
int da_gemm_bf16_ln(const float* x, const int* rows, const void* g, int g_dtype, const void* b, int b_dtype, float eps,
                    const void* w, int ldw, const void* bias, int bias_dtype, int act, void* out, int out_dtype, int ldo,
                    int M, int N, int K, void* kv_cache, const int* slot_map, int q_cols, int kv_cols, int Hkv, int D,
                    int page, void* stream);
int da_attn_decode(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks, const int* seq_lens,
                   int S, int Hq, int Hkv, int D, int page, float scale, int window, void* out, int out_ld, void* stream);
int da_attn_decode_split(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks,
                         const int* seq_lens, int S, int Hq, int Hkv, int D, int page, float scale, int window, void* out,
                         int out_ld, int n_splits, void* workspace, long workspace_bytes, void* stream);
int da_attn_prefill(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks, const int* q_start,
                    const int* seq_lens, int seq0, int n_seqs, int max_query_len, int Hq, int Hkv, int D, int page,
                    float scale, int window, void* out, int out_ld, int form, void* stream);
}

// Decode attention splits a (sequence, head) pair's keys over workgroups when the pairs alone leave most
// of the chip idle and the context is long: shares of at least 1,024 keys, as many as bring the
// workgroups to about 512, 32 at most.  The choice reads the step's shape only (pairs and the width of
// the block table), so that a recorded step keeps it.
extern "C" int da_decode_splits(int n_seqs, int n_heads, int max_blocks, int page) {
  const long by_keys = ((long)max_blocks * page) / 1024;
  const long pairs = (long)n_seqs * n_heads;
  const long by_fill = 512 / (pairs > 0 ? pairs : 1);
  long n = by_keys < by_fill ? by_keys : by_fill;
  if (n > 32) n = 32;
  return n >= 2 ? (int)n : 1;
}

// Measured on MI355X inside the model: the fused norm + product kernel wins up to 16 rows (one row tile)
// and a width of 1,024, by 10 to 15 % of a decode step; up to 8 rows (which take half the LDS, so that the
// workgroups still run side by side) up to a width of 2,048: up to 1,280 with 16 columns a workgroup, beyond
// with 32 from 5 rows on (every workgroup reads and normalises all rows again, and at a width of 1,600 that is
// 2.5 us of vector work a compute unit; with 32 columns half as many workgroups do it).  Never for a vocabulary.
extern "C" int da_can_fuse_ln(int n_rows, int K, int N) {
  const bool fits = (n_rows <= 16 && K <= 1024) || (n_rows <= 8 && K <= 2048);
  return n_rows > 0 && fits && K % 8 == 0 && N <= 16384;
}

#define DA_TRY(call) \
  do {               \
    if (call) return 1; \
  } while (0)

// out = act(norm(x[rows]) @ w.T + bias): one kernel for few rows, or the norm and then the product.
static int normed_product(const DaStep& st, const float* x, const int* rows, int n_rows, const DaNorm& nm, int K,
                          const void* w, const void* bias, int bias_dtype, int act, void* normed, void* out, int out_dtype,
                          int Nout, void* kv_cache, const int* slot_map, int q_cols, int kv_cols, int Hkv, int D, int page) {
  if (da_can_fuse_ln(n_rows, K, Nout))
    return da_gemm_bf16_ln(x, rows, nm.weight, nm.weight_dtype, nm.bias, nm.bias_dtype, nm.eps, w, K, bias, bias_dtype, act, out,
                           out_dtype, Nout, n_rows, Nout, K, kv_cache, slot_map, q_cols, kv_cols, Hkv, D, page, st.stream);
  DA_TRY(da_layernorm(x, rows, nm.weight, nm.weight_dtype, nm.bias, nm.bias_dtype, nm.eps, normed, DA_BF16, n_rows, K, st.stream));
  return da_gemm_bf16(normed, K, w, K, bias, bias_dtype, act, 0, out, out_dtype, Nout, n_rows, Nout, K, kv_cache, slot_map, q_cols,
                      kv_cols, Hkv, D, page, st.stream);
}

extern "C" int da_run_step(const DaModel* model, const DaStep* step) {
  DA_REQUIRE(model && step, "run_step: no model or no step");
  const DaModel& m = *model;
  const DaStep& st = *step;
  const int N = st.N, E = m.width;
  DA_REQUIRE(N > 0 && st.S > 0 && st.n_decode >= 0 && st.n_decode <= st.S && st.R >= 0 && E > 0 && E % 8 == 0,
             "run_step: bad sizes (N=%d S=%d decode=%d R=%d width=%d)", N, st.S, st.n_decode, st.R, E);
  DA_REQUIRE(st.n_groups >= 0 && st.n_groups <= DA_MAX_GROUPS, "run_step: %d cache groups (at most %d)", st.n_groups, DA_MAX_GROUPS);
  DA_REQUIRE(st.residual && st.norm && st.qkv && st.attn_out, "run_step: a scratch buffer is missing");

  float* x = st.residual;
  DA_TRY(da_embed(st.tokens, st.positions, m.token_table, m.token_dtype, m.pos_table, m.pos_dtype, x, N, E, m.embed_scale, st.stream));
  for (int c = 0; c < m.n_calls; ++c) {
    const DaCall& L = m.calls[c];
    DA_REQUIRE(L.group >= 0 && L.group < st.n_groups, "run_step: call %d names cache group %d of %d", c, L.group, st.n_groups);
    const int D = L.head_dim, q_cols = L.n_heads * D, kv_cols = L.n_kv_heads * D, qkv_cols = q_cols + 2 * kv_cols;
    const int g = L.group;
    // norm + q|k|v (+ bias); the new keys and values go to the cache in the product's epilogue
    DA_TRY(normed_product(st, x, nullptr, N, L.norm1, E, L.qkv_w, L.qkv_b, L.qkv_b_dtype, DA_ACT_NONE, st.norm, st.qkv, DA_BF16, qkv_cols,
                          L.write ? L.kv_cache : nullptr, L.write ? st.slot_map[g] : nullptr, L.write ? q_cols : 0,
                          L.write ? kv_cols : 0, L.write ? L.n_kv_heads : 0, L.write ? D : 0, L.write ? m.page : 0));
    // attention: the one-token sequences first, then the portions
    if (st.n_decode > 0) {
      const int splits = da_decode_splits(st.n_decode, L.n_heads, st.max_blocks[g], m.page);
      if (splits > 1) {
        DA_REQUIRE(st.decode_partial && st.decode_partial_floats >= (long)st.n_decode * L.n_heads * splits * (D + 2),
                   "run_step: the scratch of decode attention is too small");
        DA_TRY(da_attn_decode_split(st.qkv, qkv_cols, L.kv_cache, st.block_table[g], st.max_blocks[g], st.seq_lens, st.n_decode,
                                    L.n_heads, L.n_kv_heads, D, m.page, L.scale, L.window, st.attn_out, q_cols, splits,
                                    st.decode_partial, st.decode_partial_floats * 4, st.stream));
      } else {
        DA_TRY(da_attn_decode(st.qkv, qkv_cols, L.kv_cache, st.block_table[g], st.max_blocks[g], st.seq_lens, st.n_decode, L.n_heads,
                              L.n_kv_heads, D, m.page, L.scale, L.window, st.attn_out, q_cols, st.stream));
      }
    }
    if (st.S > st.n_decode)
      DA_TRY(da_attn_prefill(st.qkv, qkv_cols, L.kv_cache, st.block_table[g], st.max_blocks[g], st.q_start, st.seq_lens, st.n_decode,
                             st.S - st.n_decode, st.max_query_len, L.n_heads, L.n_kv_heads, D, m.page, L.scale, L.window, st.attn_out,
                             q_cols, 0, st.stream));
    // output projection (+ bias) into the residual stream
    DA_TRY(da_gemm_bf16(st.attn_out, q_cols, L.out_w, q_cols, L.out_b, L.out_b_dtype, DA_ACT_NONE, 1, x, DA_F32, E, N, E, q_cols, nullptr,
                        nullptr, 0, 0, 0, 0, 0, st.stream));
    if (L.has_ff) {
      DA_REQUIRE(st.ff_mid, "run_step: the feed-forward's scratch buffer is missing");
      DA_TRY(normed_product(st, x, nullptr, N, L.norm2, E, L.fc_w, L.fc_b, L.fc_b_dtype, L.act, st.norm, st.ff_mid, DA_BF16, L.inner, nullptr,
                            nullptr, 0, 0, 0, 0, 0));
      DA_TRY(da_gemm_bf16(st.ff_mid, L.inner, L.proj_w, L.inner, L.proj_b, L.proj_b_dtype, DA_ACT_NONE, 1, x, DA_F32, E, N, E, L.inner,
                          nullptr, nullptr, 0, 0, 0, 0, 0, st.stream));
    }
  }
  if (st.R == 0) return 0;
  DA_REQUIRE(st.final_norm && st.want_rows && st.logits, "run_step: rows are wanted but their buffers are missing");
  return normed_product(st, x, st.want_rows, st.R, m.final_norm, E, m.head_w, nullptr, 0, DA_ACT_NONE, st.final_norm, st.logits, DA_F32,
                        m.vocab, nullptr, nullptr, 0, 0, 0, 0, 0);
}
