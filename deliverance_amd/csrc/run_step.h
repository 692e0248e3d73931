// The model's forward pass as one call: the layer loop of a step issued from C++.
//
// `da_run_step(model, step)` runs the tokens of one step through embedding, every entry of the run order
// (norm -> q|k|v -> cache write -> attention -> output projection += ; norm -> fc + activation -> proj +=)
// and the final norm and head on the wanted rows, launching the same kernels with the same arguments as
// the parts' Python code does one by one (deliverance_amd/parts/, deliverance_amd/models/causal_lm.py),
// without a trip through the interpreter between two launches.  The reference runs its layer loop in
// one native-compiled method likewise (core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:1097-1118).
//
// It covers what the serving path of a model of standard parts is made of: bfloat16 weights, a
// LayerNorm in front of each part and none behind, attention without a rotation of q and k, a dense
// feed-forward (or none), learned or no positions at the embedding.  Models with other parts, the 32-bit
// path, the plain kernels, the debug hook and the kernel profiler go through the parts one by one.
//
// The records are plain C structs that the Python side fills through ctypes (engine/native_step.py
// declares the same fields in the same order).
#pragma once
#include <stdint.h>

#define DA_MAX_GROUPS 4

extern "C" {

typedef struct {
  const void* weight;
  const void* bias;            // may be null
  int weight_dtype, bias_dtype;
  float eps;
  int pad_;
} DaNorm;

typedef struct {
  DaNorm norm1, norm2;
  const void* qkv_w;           // [q_cols + 2 kv_cols, width] bfloat16
  const void* qkv_b;
  const void* out_w;           // [width, q_cols]
  const void* out_b;
  int qkv_b_dtype, out_b_dtype;
  int n_heads, n_kv_heads, head_dim, window;   // window 0: every earlier key
  float scale;
  int write;                   // this call writes its keys and values into the cache slot
  void* kv_cache;              // [pages, 2, n_kv_heads, page, head_dim] bfloat16
  int group;                   // which block table and slot map the cache slot goes by
  int has_ff;
  const void* fc_w;            // [inner, width]
  const void* fc_b;
  const void* proj_w;          // [width, inner]
  const void* proj_b;
  int fc_b_dtype, proj_b_dtype;
  int inner, act;
} DaCall;

typedef struct {
  int width, vocab, n_calls, page;
  const void* token_table;
  const void* pos_table;       // may be null
  int token_dtype, pos_dtype;
  float embed_scale;
  int pad_;
  DaNorm final_norm;
  const void* head_w;          // [vocab, width] bfloat16
  const DaCall* calls;
} DaModel;

typedef struct {
  int N, S, n_decode, R, max_query_len, n_groups;
  const int* tokens;
  const int* positions;
  const int* seq_of_token;
  const int* q_start;
  const int* seq_lens;
  const int* want_rows;
  const int* slot_map[DA_MAX_GROUPS];
  const int* block_table[DA_MAX_GROUPS];
  int max_blocks[DA_MAX_GROUPS];
  // scratch of the step (rows x columns): residual [N, width] f32; norm [N, width], qkv [N, widest q|k|v],
  // attn_out [N, widest q], ff_mid [N, widest inner], final_norm [R, width] bf16; logits [R, vocab] f32
  float* residual;
  void* norm;
  void* qkv;
  void* attn_out;
  void* ff_mid;
  void* final_norm;
  float* logits;
  float* decode_partial;       // for decode attention that shares a pair's keys out over workgroups
  long decode_partial_floats;
  void* stream;
} DaStep;

// 0, or non-zero with a message in da_last_error(); what was launched before a failure stays launched.
int da_run_step(const DaModel* model, const DaStep* step);

// How many shares decode attention gives a (sequence, head) pair's keys (1: none), from the step's shape only.
int da_decode_splits(int n_seqs, int n_heads, int max_blocks, int page);
// Whether the fused norm + product kernel takes a product of `n_rows` rows, inner size K and N columns.
int da_can_fuse_ln(int n_rows, int K, int N);
}
