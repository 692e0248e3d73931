// Row-wise kernels: embedding (+ learned positions), LayerNorm (optionally on gathered
// rows), and the write of new keys and values into the paged cache.
#include "common.h"
#include <stdarg.h>

static thread_local char g_error[512] = "";

extern "C" const char* da_last_error() { return g_error; }

void da_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ------------------------------------------------------------------------------------------
// x[n, :] = wte[token[n], :] * scale + wpe[pos[n], :]      (32-bit sum, 32-bit result)
// Reference: core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Model.java:42-48
// (GPT-2: scale 1; the factor is there for architectures that multiply their embeddings).
// ------------------------------------------------------------------------------------------
__global__ void embed_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                             const void* __restrict__ wte, int wte_dtype,
                             const void* __restrict__ wpe, int wpe_dtype,
                             float* __restrict__ x, int E, float scale) {
  const int n = blockIdx.x;
  const size_t trow = (size_t)tokens[n] * E;
  const size_t prow = wpe ? (size_t)positions[n] * E : 0;
  for (int i = threadIdx.x; i < E; i += blockDim.x) {
    float v = load_param(wte, wte_dtype, trow + i);
    if (scale != 1.0f) v *= scale;
    if (wpe) v += load_param(wpe, wpe_dtype, prow + i);
    x[(size_t)n * E + i] = v;
  }
}

extern "C" int da_embed(const int* tokens, const int* positions, const void* wte, int wte_dtype,
                        const void* wpe, int wpe_dtype, float* x, int N, int E, float scale, void* stream) {
  DA_REQUIRE(N >= 0 && E > 0, "embed: bad sizes N=%d E=%d", N, E);
  if (N == 0) return 0;
  int threads = E >= 256 ? 256 : (E >= 128 ? 128 : 64);
  hipLaunchKernelGGL(embed_kernel, dim3(N), dim3(threads), 0, (hipStream_t)stream, tokens, positions,
                     wte, wte_dtype, wpe, wpe_dtype, x, E, scale);
  DA_CHECK_LAUNCH("embed");
  return 0;
}

// ------------------------------------------------------------------------------------------
// dst[r, :] (+)= scale * src[rows ? rows[r] : r, :]: rows gathered, converted between 32-bit and
// bfloat16, or added into the 32-bit residual stream.  For blocks without a norm in front of a
// part, models without a final norm, norms that follow a part, and a part's output that joins the
// stream times a constant (TransformerBlock.java:260-272).
// ------------------------------------------------------------------------------------------
__global__ void copy_rows_kernel(const void* __restrict__ src, int src_dtype, const int* __restrict__ rows,
                                 void* __restrict__ dst, int dst_dtype, int E, int accumulate, float scale) {
  const int r = blockIdx.x;
  const size_t srow = (size_t)(rows ? rows[r] : r) * E, drow = (size_t)r * E;
  for (int i = threadIdx.x; i < E; i += blockDim.x) {
    const float v = load_param(src, src_dtype, srow + i) * scale;
    if (accumulate) ((float*)dst)[drow + i] += v;
    else store_out(dst, dst_dtype, drow + i, v);
  }
}

extern "C" int da_copy_rows(const void* src, int src_dtype, const int* rows, void* dst, int dst_dtype, int R,
                            int E, int accumulate, float scale, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0, "copy_rows: bad sizes R=%d E=%d", R, E);
  DA_REQUIRE(!accumulate || dst_dtype == DA_F32, "copy_rows: accumulation needs a 32-bit destination");
  if (R == 0) return 0;
  const int threads = E >= 256 ? 256 : (E >= 128 ? 128 : 64);
  hipLaunchKernelGGL(copy_rows_kernel, dim3(R), dim3(threads), 0, (hipStream_t)stream, src, src_dtype, rows, dst,
                     dst_dtype, E, accumulate, scale);
  DA_CHECK_LAUNCH("copy_rows");
  return 0;
}

// ------------------------------------------------------------------------------------------
// tokens[n] = sampled[src[n]] where src[n] >= 0: a step that is launched before the step before
// it has been read takes those tokens from that step's sampled tokens on the device.
// ------------------------------------------------------------------------------------------
__global__ void take_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ src,
                                   const int* __restrict__ sampled, int N, int n_sampled, int vocab) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const int s = src[n];
  if (s < 0 || s >= n_sampled) return;
  int t = sampled[s];
  t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);       // a row that sampled nothing must not index outside the table
  tokens[n] = t;
}

extern "C" int da_take_tokens(int* tokens, const int* src, const int* sampled, int N, int n_sampled, int vocab,
                              void* stream) {
  DA_REQUIRE(N >= 0 && n_sampled > 0 && vocab > 0, "take_tokens: bad sizes N=%d sampled=%d", N, n_sampled);
  if (N == 0) return 0;
  hipLaunchKernelGGL(take_tokens_kernel, dim3(da_ceil_div(N, 64)), dim3(64), 0, (hipStream_t)stream, tokens, src,
                     sampled, N, n_sampled, vocab);
  DA_CHECK_LAUNCH("take_tokens");
  return 0;
}

// ------------------------------------------------------------------------------------------
// Zeros over a buffer of whole 4-byte words (a kernel, so that a recorded step holds no memset node).
// ------------------------------------------------------------------------------------------
__global__ void fill_zero_kernel(uint32_t* __restrict__ p, long n_words) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) p[i] = 0u;
}

extern "C" int da_fill_zero(void* p, long n_bytes, void* stream) {
  DA_REQUIRE(n_bytes >= 0 && n_bytes % 4 == 0 && (uintptr_t)p % 4 == 0, "fill_zero: %ld bytes are not whole words", n_bytes);
  if (n_bytes == 0) return 0;
  const long words = n_bytes / 4;
  const int blocks = (int)(words / 256 < 1 ? 1 : (words / 256 > 2048 ? 2048 : words / 256));
  hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)p, words);
  DA_CHECK_LAUNCH("fill_zero");
  return 0;
}

// ------------------------------------------------------------------------------------------
// Fixed-size state of the step's sequences, as rows of 4-byte words (any dtype).
//   gather:  out[n, :] = state[slot[seq_of_token[n]], :]   (zeros where the sequence has no slot: a padding row)
//   scatter: state[slot[s], :] = rows[q_start[s+1] - 1, :] for every sequence s that has a slot and brings rows
// A mixer with state reads the first before it walks its rows and calls the second with what each row
// leaves behind: the state of a portion's last row is the request's state after the step.
// ------------------------------------------------------------------------------------------
__global__ void state_gather_kernel(const uint32_t* __restrict__ state, const int* __restrict__ slots,
                                    const int* __restrict__ seq_of_token, uint32_t* __restrict__ out,
                                    int n_slots, int words) {
  const int n = blockIdx.x;
  const int slot = slots[seq_of_token[n]];
  const bool has = slot >= 0 && slot < n_slots;
  for (int i = threadIdx.x; i < words; i += blockDim.x)
    out[(size_t)n * words + i] = has ? state[(size_t)slot * words + i] : 0u;
}

__global__ void state_scatter_kernel(uint32_t* __restrict__ state, const int* __restrict__ slots,
                                     const int* __restrict__ q_start, const uint32_t* __restrict__ rows,
                                     int n_slots, int words) {
  const int s = blockIdx.x;
  const int slot = slots[s], first = q_start[s], last = q_start[s + 1] - 1;
  if (slot < 0 || slot >= n_slots || last < first) return;
  for (int i = threadIdx.x; i < words; i += blockDim.x) state[(size_t)slot * words + i] = rows[(size_t)last * words + i];
}

extern "C" int da_state_gather(const void* state, const int* slots, const int* seq_of_token, void* out, int N,
                               int n_slots, int row_bytes, void* stream) {
  DA_REQUIRE(N >= 0 && n_slots > 0 && row_bytes > 0 && row_bytes % 4 == 0, "state_gather: bad sizes (N=%d, %d slots, rows of %d bytes)",
             N, n_slots, row_bytes);
  if (N == 0) return 0;
  hipLaunchKernelGGL(state_gather_kernel, dim3(N), dim3(row_bytes / 4 >= 256 ? 256 : 64), 0, (hipStream_t)stream,
                     (const uint32_t*)state, slots, seq_of_token, (uint32_t*)out, n_slots, row_bytes / 4);
  DA_CHECK_LAUNCH("state_gather");
  return 0;
}

extern "C" int da_state_scatter(void* state, const int* slots, const int* q_start, const void* rows, int S,
                                int n_slots, int row_bytes, void* stream) {
  DA_REQUIRE(S >= 0 && n_slots > 0 && row_bytes > 0 && row_bytes % 4 == 0, "state_scatter: bad sizes (S=%d, %d slots, rows of %d bytes)",
             S, n_slots, row_bytes);
  if (S == 0) return 0;
  hipLaunchKernelGGL(state_scatter_kernel, dim3(S), dim3(row_bytes / 4 >= 256 ? 256 : 64), 0, (hipStream_t)stream,
                     (uint32_t*)state, slots, q_start, (const uint32_t*)rows, n_slots, row_bytes / 4);
  DA_CHECK_LAUNCH("state_scatter");
  return 0;
}

// ------------------------------------------------------------------------------------------
// LayerNorm over rows of 32-bit x; one wave per row; mean and centred variance in 32-bit.
//   y = (x - mean) / sqrt(var + eps) * w + b        (var biased, eps inside the root)
// Reference: core/src/main/java/io/teknek/deliverance/generator/LayerNorm.java:127-150
// `rows` (optional) gathers: output row r is the norm of input row rows[r].
// ------------------------------------------------------------------------------------------
__global__ void layernorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                 const void* __restrict__ w, int w_dtype,
                                 const void* __restrict__ b, int b_dtype, float eps,
                                 void* __restrict__ y, int y_dtype, int R, int E) {
  const int wave = threadIdx.x / DA_WAVE, lane = threadIdx.x % DA_WAVE;
  const int r = blockIdx.x * (blockDim.x / DA_WAVE) + wave;
  if (r >= R) return;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * E;
  float s = 0.f;
  for (int i = lane; i < E; i += DA_WAVE) s += xr[i];
  const float mean = wave_sum(s) / (float)E;
  float q = 0.f;
  for (int i = lane; i < E; i += DA_WAVE) {
    float d = xr[i] - mean;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(wave_sum(q) / (float)E + eps);
  for (int i = lane; i < E; i += DA_WAVE) {
    float v = (xr[i] - mean) * inv * load_param(w, w_dtype, i);
    if (b) v += load_param(b, b_dtype, i);
    store_out(y, y_dtype, (size_t)r * E + i, v);
  }
}

__device__ __forceinline__ float4 load_param4(const void* p, int dtype, int i) {
  if (dtype == DA_BF16) {
    const uint2 u = *(const uint2*)((const bf16_t*)p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
  return *(const float4*)((const float*)p + i);
}

// The same norm with the whole row held in registers: every load of the row is in flight at
// once, which is what counts when a step has a handful of rows.  E a multiple of 4, E <= 256*VPL.
// A workgroup is one wavefront (few rows: as many compute units as rows) or four (many rows: fewer,
// fuller workgroups).
// Loads come back in the order they were asked for: the row first, then gain and bias, as raw bits
// that are converted where they are used (a conversion right after its load, or a load inside a
// branch, is waited for on the spot).  PBF16: gain and bias are bfloat16 (else 32-bit).
template <int VPL, bool PBF16>
__global__ void __launch_bounds__(4 * DA_WAVE)
layernorm_row_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                     const void* __restrict__ w, const void* __restrict__ b,
                     float eps, void* __restrict__ y, int y_dtype, int R, int E) {
  const int lane = threadIdx.x % DA_WAVE;
  const int r = blockIdx.x * (blockDim.x / DA_WAVE) + threadIdx.x / DA_WAVE;
  if (r >= R) return;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * E;
  // every load of the row, of the gain and of the bias is asked for at once (past the row's end
  // the row's start is read and left out of the sums), before anything is reduced
  float4 v[VPL];
  uint4 graw[VPL], braw[VPL];           // bfloat16: .x and .y hold the four values
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4;
    v[i] = *(const float4*)(xr + (c < E ? c : 0));
  }
  const void* bsrc = b ? b : w;         // without a bias the gain is read twice and dropped
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4, cc = c < E ? c : 0;
    if (PBF16) {
      const uint2 g2 = *(const uint2*)((const bf16_t*)w + cc), b2 = *(const uint2*)((const bf16_t*)bsrc + cc);
      graw[i] = make_uint4(g2.x, g2.y, 0, 0);
      braw[i] = make_uint4(b2.x, b2.y, 0, 0);
    } else {
      graw[i] = *(const uint4*)((const float*)w + cc);
      braw[i] = *(const uint4*)((const float*)bsrc + cc);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < VPL; ++i)
    s += ((lane + i * DA_WAVE) * 4 < E ? 1.f : 0.f) * ((v[i].x + v[i].y) + (v[i].z + v[i].w));
  const float mean = wave_sum(s) / (float)E;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4;
    if (c < E) {
      const float d0 = v[i].x - mean, d1 = v[i].y - mean, d2 = v[i].z - mean, d3 = v[i].w - mean;
      q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
  }
  const float inv = 1.0f / sqrtf(wave_sum(q) / (float)E + eps);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4;
    if (c < E) {
      float4 g, bb;
      if (PBF16) {
        g = make_float4(__uint_as_float(graw[i].x << 16), __uint_as_float(graw[i].x & 0xffff0000u),
                        __uint_as_float(graw[i].y << 16), __uint_as_float(graw[i].y & 0xffff0000u));
        bb = make_float4(__uint_as_float(braw[i].x << 16), __uint_as_float(braw[i].x & 0xffff0000u),
                         __uint_as_float(braw[i].y << 16), __uint_as_float(braw[i].y & 0xffff0000u));
      } else {
        g = make_float4(__uint_as_float(graw[i].x), __uint_as_float(graw[i].y), __uint_as_float(graw[i].z), __uint_as_float(graw[i].w));
        bb = make_float4(__uint_as_float(braw[i].x), __uint_as_float(braw[i].y), __uint_as_float(braw[i].z), __uint_as_float(braw[i].w));
      }
      if (!b) bb = make_float4(0.f, 0.f, 0.f, 0.f);
      const float4 o = make_float4((v[i].x - mean) * inv * g.x + bb.x, (v[i].y - mean) * inv * g.y + bb.y,
                                   (v[i].z - mean) * inv * g.z + bb.z, (v[i].w - mean) * inv * g.w + bb.w);
      if (y_dtype == DA_BF16) {
        uint2 u;
        u.x = (uint32_t)f32_to_bf16(o.x) | ((uint32_t)f32_to_bf16(o.y) << 16);
        u.y = (uint32_t)f32_to_bf16(o.z) | ((uint32_t)f32_to_bf16(o.w) << 16);
        *(uint2*)((bf16_t*)y + (size_t)r * E + c) = u;
      } else {
        *(float4*)((float*)y + (size_t)r * E + c) = o;
      }
    }
  }
}

extern "C" int da_layernorm(const float* x, const int* rows, const void* w, int w_dtype,
                            const void* b, int b_dtype, float eps, void* y, int y_dtype, int R,
                            int E, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0, "layernorm: bad sizes R=%d E=%d", R, E);
  DA_REQUIRE(eps > 0.f, "layernorm: eps must be > 0");
  if (R == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                       (!b || (uintptr_t)b % 16 == 0);
  const int wpb = R >= 512 ? 4 : 1;      // wavefronts (rows) per workgroup
  const bool same = (!b || b_dtype == w_dtype) && (w_dtype == DA_BF16 || w_dtype == DA_F32);   // gain and bias alike
  if (E % 4 == 0 && E <= 2048 && aligned && same) {
#define LN_LAUNCH(V)                                                                                                \
  do {                                                                                                              \
    if (w_dtype == DA_BF16)                                                                                         \
      hipLaunchKernelGGL((layernorm_row_kernel<V, true>), dim3(da_ceil_div(R, wpb)), dim3(wpb * DA_WAVE), 0, st, x, \
                         rows, w, b, eps, y, y_dtype, R, E);                                                        \
    else                                                                                                            \
      hipLaunchKernelGGL((layernorm_row_kernel<V, false>), dim3(da_ceil_div(R, wpb)), dim3(wpb * DA_WAVE), 0, st, x, \
                         rows, w, b, eps, y, y_dtype, R, E);                                                        \
  } while (0)
    if (E <= 256) LN_LAUNCH(1);
    else if (E <= 512) LN_LAUNCH(2);
    else if (E <= 1024) LN_LAUNCH(4);
    else LN_LAUNCH(8);
#undef LN_LAUNCH
  } else {
    const int waves = 4;
    hipLaunchKernelGGL(layernorm_kernel, dim3(da_ceil_div(R, waves)), dim3(waves * DA_WAVE), 0, st, x, rows, w,
                       w_dtype, b, b_dtype, eps, y, y_dtype, R, E);
  }
  DA_CHECK_LAUNCH("layernorm");
  return 0;
}

// ------------------------------------------------------------------------------------------
// Keys and values of the step's tokens go to their cache rows.
// qkv: [N, ld] rows holding q | k | v; k starts at column k_off, v at v_off, each Hkv*D wide.
// One cache slot (one layer's pages): [n_pages][2][Hkv][page * D], keys row-major, values
// dimension-major (see common.h); slot_map[n] is page_id * page + row, or -1 for a token whose
// keys are not kept.
// Reference: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:315-336
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ qkv, int ld, int k_off, int v_off,
                                T* __restrict__ cache, const int* __restrict__ slot_map, int Hkv,
                                int D, int page) {
  const int n = blockIdx.x;
  const int slot = slot_map[n];
  if (slot < 0) return;
  const int pg = slot / page, row = slot % page;
  const int W = Hkv * D;
  for (int i = threadIdx.x; i < 2 * W; i += blockDim.x) {
    const int kv = i / W, c = i % W, h = c / D, d = c % D;
    const T v = qkv[(size_t)n * ld + (kv ? v_off : k_off) + c];
    if (kv) cache[cache_v_base(pg, h, Hkv, page, D) + (long long)d * page + row] = v;
    else cache[cache_k_row(pg, h, row, Hkv, page, D) + d] = v;
  }
}

// The same for bfloat16 and many tokens: a workgroup takes 16 consecutive tokens.  Keys go over in
// 16-byte pieces.  Where the 16 tokens fill 16 consecutive, aligned rows of one page (a prompt
// portion that starts on such a boundary), a value column's 16 entries are one 32-byte run in the
// dimension-major page and are stored as such; otherwise entry by entry.
#define KVW_ROWS 16
__global__ void __launch_bounds__(256)
kv_write_rows_kernel(const bf16_t* __restrict__ qkv, int ld, int k_off, int v_off, bf16_t* __restrict__ cache,
                     const int* __restrict__ slot_map, int N, int Hkv, int D, int page) {
  __shared__ int slots[KVW_ROWS];
  __shared__ int run;
  const int n0 = blockIdx.x * KVW_ROWS;
  if (threadIdx.x < KVW_ROWS) slots[threadIdx.x] = n0 + threadIdx.x < N ? slot_map[n0 + threadIdx.x] : -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    int ok = slots[0] >= 0 && slots[0] % KVW_ROWS == 0;
    for (int i = 1; i < KVW_ROWS; ++i) ok = ok && slots[i] == slots[0] + i;
    run = ok;
  }
  __syncthreads();
  const int W = Hkv * D, chunks = W / 8;
  // blockIdx.y splits the columns, so that few tokens still fill the chip
  const int t = threadIdx.x + blockIdx.y * blockDim.x, stride = blockDim.x * gridDim.y;
  // keys: rows of 16-byte pieces
  for (int e = t; e < KVW_ROWS * chunks; e += stride) {
    const int i = e / chunks, c = (e % chunks) * 8, slot = slots[i];
    if (slot < 0) continue;
    const int h = c / D, d = c % D;
    *(uint4*)(cache + cache_k_row(slot / page, h, slot % page, Hkv, page, D) + d) =
        *(const uint4*)(qkv + (size_t)(n0 + i) * ld + k_off + c);
  }
  // values: a thread takes a column (head, dimension) of the 16 tokens
  for (int c = t; c < W; c += stride) {
    const int h = c / D, d = c % D;
    bf16_t v[KVW_ROWS];
#pragma unroll
    for (int i = 0; i < KVW_ROWS; ++i) v[i] = slots[i] >= 0 ? qkv[(size_t)(n0 + i) * ld + v_off + c] : (bf16_t)0;
    if (run) {
      bf16_t* dst = cache + cache_v_base(slots[0] / page, h, Hkv, page, D) + (long long)d * page + slots[0] % page;
      uint32_t u[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) u[i] = (uint32_t)v[2 * i] | ((uint32_t)v[2 * i + 1] << 16);
      *(uint4*)dst = make_uint4(u[0], u[1], u[2], u[3]);
      *(uint4*)(dst + 8) = make_uint4(u[4], u[5], u[6], u[7]);
    } else {
#pragma unroll
      for (int i = 0; i < KVW_ROWS; ++i)
        if (slots[i] >= 0)
          cache[cache_v_base(slots[i] / page, h, Hkv, page, D) + (long long)d * page + slots[i] % page] = v[i];
    }
  }
}

extern "C" int da_kv_write(const void* qkv, int dtype, int ld, int k_off, int v_off, void* cache,
                           const int* slot_map, int N, int Hkv, int D, int page, void* stream) {
  DA_REQUIRE(N >= 0 && Hkv > 0 && D > 0 && page > 0, "kv_write: bad sizes");
  DA_REQUIRE(k_off >= 0 && v_off >= 0 && k_off + Hkv * D <= ld && v_off + Hkv * D <= ld,
             "kv_write: k/v columns [%d,%d)+%d exceed the row length %d", k_off, v_off, Hkv * D, ld);
  if (N == 0) return 0;
  const int threads = 256;
  const bool vec = dtype == DA_BF16 && N >= 256 && D % 8 == 0 && page % KVW_ROWS == 0 && ld % 8 == 0 &&
                   k_off % 8 == 0 && ((uintptr_t)qkv % 16 == 0) && ((uintptr_t)cache % 16 == 0);
  if (vec)
    hipLaunchKernelGGL(kv_write_rows_kernel, dim3(da_ceil_div(N, KVW_ROWS), da_ceil_div(Hkv * D, 256)), dim3(threads), 0, (hipStream_t)stream,
                       (const bf16_t*)qkv, ld, k_off, v_off, (bf16_t*)cache, slot_map, N, Hkv, D, page);
  else if (dtype == DA_BF16)
    hipLaunchKernelGGL(kv_write_kernel<bf16_t>, dim3(N), dim3(threads), 0, (hipStream_t)stream,
                       (const bf16_t*)qkv, ld, k_off, v_off, (bf16_t*)cache, slot_map, Hkv, D, page);
  else
    hipLaunchKernelGGL(kv_write_kernel<float>, dim3(N), dim3(threads), 0, (hipStream_t)stream,
                       (const float*)qkv, ld, k_off, v_off, (float*)cache, slot_map, Hkv, D, page);
  DA_CHECK_LAUNCH("kv_write");
  return 0;
}
