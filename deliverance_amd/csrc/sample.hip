// Sampling on the device, one workgroup per row of logits.
//
// Greedy: arg-max, the first maximum wins (core/src/main/java/io/teknek/deliverance/model/
// AbstractGeneratorSampler.java:135-151,161-173).
// Temperature: v = logit / T; candidates in descending order of v (ties by ascending index,
// the order a stable sort gives); keep the first k; keep the nucleus whose cumulative
// probability first reaches p; walk the kept list with pick = u * total
// (AbstractGeneratorSampler.java:266-323).  "Exclude top choices": among tokens whose
// probability exceeds the threshold, take the least likely one
// (core/.../model/ExcludeTopChoicePicker.java:42-85).
//
// No sort is materialised.  A prefix of the sorted order is (tau, r): every key above tau
// plus the first r entries (by index) whose key equals tau.  The prefix that reaches a given
// mass or count is found by a bitwise search over the 32-bit ordered key of a float, each
// probe being one pass over the row with a reduction in a fixed order, so equal inputs give
// equal tokens.  Weights are exp(v - max) in 32-bit, summed in 64-bit.
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / DA_WAVE)

struct SampleRow {
  float temperature;    // 0: greedy
  int top_k;            // candidates kept, 0: all
  float top_p;          // 0: off
  int uniform_top_p;    // pick uniformly inside the nucleus
  float u;              // the uniform draw for the pick
  float xtc_threshold;  // 0: off
  int xtc_active;       // the draw fell inside the xtc probability
  int pad;
};

__device__ __forceinline__ uint32_t ordered_key(float v) {
  uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

struct Reducer {
  double* d;   // [SAMPLE_WAVES]
  int* i;      // [SAMPLE_WAVES]
  float* f;    // [SAMPLE_WAVES]
};

__device__ void block_sum(const Reducer& R, double& mass, int& count) {
  mass = wave_sum_d(mass);
  count = wave_sum_i(count);
  const int wave = threadIdx.x / DA_WAVE, lane = threadIdx.x % DA_WAVE;
  __syncthreads();
  if (lane == 0) { R.d[wave] = mass; R.i[wave] = count; }
  __syncthreads();
  double m = 0.0; int c = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) { m += R.d[w]; c += R.i[w]; }
  mass = m; count = c;
}

// best (value, index): larger value wins, then smaller index (or larger value loses when
// `want_min`: smaller value wins, then smaller index).
__device__ void block_best(const Reducer& R, float& v, int& idx, bool want_min) {
  auto better = [&](float a, int ai, float b, int bi) {
    if (ai < 0) return false;
    if (bi < 0) return true;
    if (a != b) return want_min ? a < b : a > b;
    return ai < bi;
  };
  wave_best(v, idx, better);
  const int wave = threadIdx.x / DA_WAVE, lane = threadIdx.x % DA_WAVE;
  __syncthreads();
  if (lane == 0) { R.f[wave] = v; R.i[wave] = idx; }
  __syncthreads();
  float bv = R.f[0]; int bi = R.i[0];
  for (int w = 1; w < SAMPLE_WAVES; ++w)
    if (better(R.f[w], R.i[w], bv, bi)) { bv = R.f[w]; bi = R.i[w]; }
  v = bv; idx = bi;
}

struct RowView {
  const float* row;
  int V;
  float T;      // divisor (1 when the raw logits are meant)
  float vmax;   // max of row[i] / T
  __device__ float value(int i) const { return row[i] / T; }
};

// mass and count of entries whose key is >= tau
__device__ void ge_stats(const RowView& rv, const Reducer& R, uint32_t tau, double& mass, int& count) {
  double m = 0.0; int c = 0;
  for (int i = threadIdx.x; i < rv.V; i += SAMPLE_THREADS) {
    const float v = rv.value(i);
    if (ordered_key(v) >= tau) { m += (double)expf(v - rv.vmax); ++c; }
  }
  block_sum(R, m, c);
  mass = m; count = c;
}

struct Prefix {
  uint32_t tau;
  int r;           // entries with key == tau that belong to the prefix (>= 1)
  double mass_gt;  // mass of keys above tau
  int count_gt;
  float w;         // weight of one entry at tau
  __device__ double mass() const { return mass_gt + (double)r * (double)w; }
  __device__ int count() const { return count_gt + r; }
};

// The shortest prefix of the sorted order whose mass reaches `target_mass` (by_mass) or whose
// length reaches `target_count`, cut to `bound` when it would pass it.
__device__ Prefix find_prefix(const RowView& rv, const Reducer& R, bool by_mass, double target_mass,
                              int target_count, const Prefix* bound) {
  uint32_t tau = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t t = tau | (1u << bit);
    double m; int c;
    ge_stats(rv, R, t, m, c);
    if (by_mass ? (m >= target_mass) : (c >= target_count)) tau = t;
  }
  if (bound && tau < bound->tau) tau = bound->tau;
  Prefix p;
  p.tau = tau;
  double m_ge, m_gt; int c_ge, c_gt;
  ge_stats(rv, R, tau, m_ge, c_ge);
  if (tau == 0xffffffffu) { m_gt = 0.0; c_gt = 0; }
  else ge_stats(rv, R, tau + 1u, m_gt, c_gt);
  p.mass_gt = m_gt;
  p.count_gt = c_gt;
  p.w = expf(key_value(tau) - rv.vmax);
  int ties = c_ge - c_gt;
  if (bound && tau == bound->tau) ties = bound->r;
  int r;
  if (by_mass) {
    const double need = target_mass - m_gt;
    r = (p.w > 0.f) ? (int)ceil(need / (double)p.w) : ties;
  } else {
    r = target_count - c_gt;
  }
  if (r < 1) r = 1;
  if (r > ties) r = ties;
  if (r < 1) r = 1;
  p.r = r;
  return p;
}

// index of the r-th entry (1-based, ascending index) whose key equals tau
__device__ int nth_with_key(const RowView& rv, uint32_t tau, int r, int* counts, int* found) {
  const int chunk = (rv.V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int b = threadIdx.x * chunk;
  const int e = (b + chunk < rv.V) ? b + chunk : rv.V;
  int c = 0;
  for (int i = b; i < e; ++i) c += (ordered_key(rv.value(i)) == tau);
  __syncthreads();
  counts[threadIdx.x] = c;
  if (threadIdx.x == 0) { found[0] = -1; }
  __syncthreads();
  if (threadIdx.x == 0) {
    int left = r, owner = -1;
    for (int t = 0; t < SAMPLE_THREADS; ++t) {
      if (left <= counts[t]) { owner = t; break; }
      left -= counts[t];
    }
    found[1] = owner;
    found[2] = left;
  }
  __syncthreads();
  if (threadIdx.x == found[1]) {
    int left = found[2];
    for (int i = b; i < e; ++i)
      if (ordered_key(rv.value(i)) == tau && --left == 0) { found[0] = i; break; }
  }
  __syncthreads();
  return found[0];
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int ldl, int V, const SampleRow* __restrict__ params,
              int* __restrict__ tokens) {
  __shared__ double red_d[SAMPLE_WAVES];
  __shared__ int red_i[SAMPLE_WAVES];
  __shared__ float red_f[SAMPLE_WAVES];
  __shared__ int counts[SAMPLE_THREADS];
  __shared__ int found[4];
  const Reducer R{red_d, red_i, red_f};
  const int r = blockIdx.x;
  const SampleRow sp = params[r];
  const float* row = logits + (size_t)r * ldl;

  // the largest entry (the lowest index among equals): ARGMAX_LOADS loads in flight per thread, from
  // clamped places, so that a vocabulary of 50,000 is crossed in two memory round trips
  constexpr int ARGMAX_LOADS = 25;
  float best = -INFINITY; int besti = -1;
  for (int i0 = threadIdx.x; i0 < V; i0 += ARGMAX_LOADS * SAMPLE_THREADS) {
    float v[ARGMAX_LOADS];
#pragma unroll
    for (int u = 0; u < ARGMAX_LOADS; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      v[u] = row[i < V ? i : V - 1];
    }
#pragma unroll
    for (int u = 0; u < ARGMAX_LOADS; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      if (i < V && (besti < 0 || v[u] > best)) { best = v[u]; besti = i; }
    }
  }
  block_best(R, best, besti, false);
  const bool xtc = sp.xtc_threshold != 0.f;
  if (sp.temperature == 0.f && !xtc) {
    if (threadIdx.x == 0) tokens[r] = besti;
    return;
  }
  RowView rv;
  rv.row = row; rv.V = V;
  rv.T = sp.temperature == 0.f ? 1.0f : sp.temperature;
  rv.vmax = best / rv.T;

  if (xtc) {
    // probability of entry i is exp(v_i - vmax) / total
    int chosen = -1;
    if (sp.xtc_active) {
      double total; int n;
      ge_stats(rv, R, 0u, total, n);
      float lo = INFINITY; int loi = -1;
      for (int i = threadIdx.x; i < V; i += SAMPLE_THREADS) {
        const float v = rv.value(i);
        const float prob = (float)((double)expf(v - rv.vmax) / total);
        if (prob > sp.xtc_threshold && (loi < 0 || v < lo)) { lo = v; loi = i; }
      }
      block_best(R, lo, loi, true);
      chosen = loi;
    }
    if (threadIdx.x == 0) tokens[r] = chosen >= 0 ? chosen : besti;
    return;
  }

  Prefix kept;            // the candidates: everything, or the first k
  bool have = false;
  if (sp.top_k > 0 && sp.top_k < V) {
    kept = find_prefix(rv, R, false, 0.0, sp.top_k, nullptr);
    have = true;
  }
  double total;
  if (have) total = kept.mass();
  else { int n; ge_stats(rv, R, 0u, total, n); }
  if (sp.top_p > 0.f) {
    kept = find_prefix(rv, R, true, (double)sp.top_p * total, 0, have ? &kept : nullptr);
    have = true;
    total = kept.mass();
    if (sp.uniform_top_p) {
      const int n = kept.count();
      int pick = (int)(sp.u * (float)n);
      if (pick > n - 1) pick = n - 1;
      const Prefix at = find_prefix(rv, R, false, 0.0, pick + 1, &kept);
      const int tok = nth_with_key(rv, at.tau, at.r, counts, found);
      if (threadIdx.x == 0) tokens[r] = tok >= 0 ? tok : besti;
      return;
    }
  }
  const Prefix at = find_prefix(rv, R, true, (double)sp.u * total, 0, have ? &kept : nullptr);
  const int tok = nth_with_key(rv, at.tau, at.r, counts, found);
  if (threadIdx.x == 0) tokens[r] = tok >= 0 ? tok : besti;
}

extern "C" int da_sample(const float* logits, int ldl, int R, int V, const void* params, int* tokens,
                         void* stream) {
  DA_REQUIRE(R >= 0 && V > 0 && ldl >= V, "sample: bad sizes R=%d V=%d ld=%d", R, V, ldl);
  if (R == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, logits, ldl, V,
                     (const SampleRow*)params, tokens);
  DA_CHECK_LAUNCH("sample");
  return 0;
}

// ------------------------------------------------------------------------------------------
// The n most likely tokens of each row with logprob = v - log sum exp(v)
// (AbstractGeneratorSampler.java:137-155,247-254), v = logit / T (T = 1 for greedy rows).
// One pass per rank: the best entry strictly after the previous one in (value desc, index asc).
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(SAMPLE_THREADS)
top_logprobs_kernel(const float* __restrict__ logits, int ldl, int V, const SampleRow* __restrict__ params,
                    int n, int* __restrict__ out_idx, float* __restrict__ out_lp) {
  __shared__ double red_d[SAMPLE_WAVES];
  __shared__ int red_i[SAMPLE_WAVES];
  __shared__ float red_f[SAMPLE_WAVES];
  const Reducer R{red_d, red_i, red_f};
  const int r = blockIdx.x;
  const float T = params[r].temperature == 0.f ? 1.0f : params[r].temperature;
  RowView rv;
  rv.row = logits + (size_t)r * ldl; rv.V = V; rv.T = T;
  float best = -INFINITY; int besti = -1;
  for (int i = threadIdx.x; i < V; i += SAMPLE_THREADS) {
    const float v = rv.value(i);
    if (besti < 0 || v > best) { best = v; besti = i; }
  }
  block_best(R, best, besti, false);
  rv.vmax = best;
  double total; int cnt;
  ge_stats(rv, R, 0u, total, cnt);
  const float lse = best + (float)log(total);
  float pv = best; int pi = besti;
  for (int k = 0; k < n; ++k) {
    if (k > 0) {
      float bv = -INFINITY; int bi = -1;
      for (int i = threadIdx.x; i < V; i += SAMPLE_THREADS) {
        const float v = rv.value(i);
        const bool after = (v < pv) || (v == pv && i > pi);
        if (after && (bi < 0 || v > bv)) { bv = v; bi = i; }
      }
      block_best(R, bv, bi, false);
      pv = bv; pi = bi;
    }
    if (threadIdx.x == 0) {
      out_idx[(size_t)r * n + k] = pi;
      out_lp[(size_t)r * n + k] = pi >= 0 ? pv - lse : -INFINITY;
    }
    if (pi < 0) { pv = -INFINITY; }
  }
}

extern "C" int da_top_logprobs(const float* logits, int ldl, int R, int V, const void* params, int n,
                               int* out_idx, float* out_lp, void* stream) {
  DA_REQUIRE(R >= 0 && V > 0 && ldl >= V && n > 0 && n <= V, "top_logprobs: bad sizes R=%d V=%d n=%d", R, V, n);
  if (R == 0) return 0;
  hipLaunchKernelGGL(top_logprobs_kernel, dim3(R), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, logits, ldl,
                     V, (const SampleRow*)params, n, out_idx, out_lp);
  DA_CHECK_LAUNCH("top_logprobs");
  return 0;
}
