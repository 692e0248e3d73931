// Plain paged attention: one wavefront per (token, query head), any mix of prompt rows and
// decode rows.  It is the attention of the true 32-bit path and the reference beside the
// MFMA prefill kernel and the split-context decode kernel.
//
// For the token at position p of its sequence, head h:
//   s_j = (q . k_j) * scale   for j in [lo, p],  lo = 0 or p - window + 1
//   w   = softmax(s)          (max, exp, sum in 32-bit)
//   o   = sum_j w_j v_j
// Reference: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:481-491,
// 512-527 and the online-softmax recurrence of
// native/src/main/resources/decode_paged_attention_f32.wgsl:31-65.
//
// Keys are walked in chunks of 64 starting at lo, so the order of the sums depends only on
// the token's own position, never on how the step was cut or what else is in the batch.
#include "common.h"

#define MAX_D 256

template <typename T>
__global__ void __launch_bounds__(DA_WAVE)
attn_ref_kernel(const T* __restrict__ q, int q_ld, const T* __restrict__ cache,
                const int* __restrict__ block_table, int max_blocks,
                const int* __restrict__ seq_of_token, const int* __restrict__ positions,
                int Hq, int Hkv, int D, int page, float scale, int window,
                T* __restrict__ out, int out_ld) {
  __shared__ float qs[MAX_D];
  __shared__ float ps[DA_WAVE];
  __shared__ long long voff[DA_WAVE];
  const int lane = threadIdx.x;
  const int n = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const int hk = h / (Hq / Hkv);
  const int p = positions[n];
  const int* bt = block_table + (size_t)seq_of_token[n] * max_blocks;

  for (int d = lane; d < D; d += DA_WAVE) qs[d] = to_f32(q[(size_t)n * q_ld + h * D + d]);
  __syncthreads();

  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / DA_WAVE];
#pragma unroll
  for (int i = 0; i < MAX_D / DA_WAVE; ++i) acc[i] = 0.f;

  for (int c0 = lo; c0 <= p; c0 += DA_WAVE) {
    const int key = c0 + lane;
    // a row whose sequence has no page there (a padding row of a fixed-shape step) sees nothing
    const bool valid = key <= p && bt[key / page] >= 0;
    float s = -INFINITY;
    if (valid) {
      const long long pg = bt[key / page];
      const int row = key % page;
      const T* kr = cache + cache_k_row(pg, hk, row, Hkv, page, D);
      voff[lane] = cache_v_base(pg, hk, Hkv, page, D) + row;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float e = valid ? expf(s - m_new) : 0.f;
    // 0 on the first chunk that shows a key (m = -inf); 1 while no key has been seen at all (a
    // padding row of a fixed-shape step: -inf - -inf would be NaN, and NaN * 0 stays NaN)
    const float alpha = m_new == -INFINITY ? 1.f : expf(m - m_new);
    l = l * alpha + wave_sum(e);
    m = m_new;
    ps[lane] = e;
    __syncthreads();
    const int cnt = (p - c0 + 1 < DA_WAVE) ? p - c0 + 1 : DA_WAVE;
#pragma unroll
    for (int i = 0; i < MAX_D / DA_WAVE; ++i) {
      const int d = lane + i * DA_WAVE;
      if (d < D) {
        float a = acc[i] * alpha;
        for (int j = 0; j < cnt; ++j) {
          const float pj = ps[j];                  // 0 for a key that is not seen: its row is not read
          if (pj != 0.f) a = fmaf(pj, to_f32(cache[voff[j] + (long long)d * page]), a);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int i = 0; i < MAX_D / DA_WAVE; ++i) {
    const int d = lane + i * DA_WAVE;
    if (d < D) from_f32(&out[(size_t)n * out_ld + h * D + d], acc[i] * inv);
  }
}

extern "C" int da_attn_ref(const void* q, int q_ld, const void* cache, int dtype,
                           const int* block_table, int max_blocks, const int* seq_of_token,
                           const int* positions, int N, int Hq, int Hkv, int D, int page, float scale,
                           int window, void* out, int out_ld, void* stream) {
  DA_REQUIRE(N >= 0 && Hq > 0 && Hkv > 0 && D > 0 && page > 0, "attn_ref: bad sizes");
  DA_REQUIRE(Hq % Hkv == 0, "attn_ref: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(D <= MAX_D, "attn_ref: head size %d exceeds %d", D, MAX_D);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * D, "attn_ref: row lengths too small");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_ref: bad window or block table");
  if (N == 0) return 0;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(attn_ref_kernel<bf16_t>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream,
                       (const bf16_t*)q, q_ld, (const bf16_t*)cache, block_table, max_blocks, seq_of_token,
                       positions, Hq, Hkv, D, page, scale, window, (bf16_t*)out, out_ld);
  else
    hipLaunchKernelGGL(attn_ref_kernel<float>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream,
                       (const float*)q, q_ld, (const float*)cache, block_table, max_blocks, seq_of_token,
                       positions, Hq, Hkv, D, page, scale, window, (float*)out, out_ld);
  DA_CHECK_LAUNCH("attn_ref");
  return 0;
}
