"""Python faces of the HIP kernels.

Each function checks on the host that the operands have the shapes, dtypes and layout the
kernel and its grid assume, then launches on torch's current stream.  Nothing here falls
back to a library or to the CPU: a missing kernel library is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build
from ..profiler import KernelProfiler

F32, BF16 = 0, 1
MAX_HEAD_DIM = 256          # what the plain attention kernel takes; the matrix-core kernels: multiples of 16 up to it
ACTIVATIONS = {None: 0, "none": 0, "gelu_new": 1, "gelu_pytorch_tanh": 1, "gelu": 2, "relu": 3, "silu": 4}


class KernelError(RuntimeError):
    pass


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, found {t.dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


_PINNED_STREAM = None


def _stream():
    if _PINNED_STREAM is not None:
        return _PINNED_STREAM
    return torch.cuda.current_stream().cuda_stream


class pinned_stream:
    """Inside this context every kernel goes to the stream that was current on entry, without asking
    torch again for each launch (a model step launches about a hundred kernels)."""

    def __enter__(self):
        global _PINNED_STREAM
        self._old = _PINNED_STREAM
        _PINNED_STREAM = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _PINNED_STREAM
        _PINNED_STREAM = self._old
        return False


def _check(rc: int):
    if rc != 0:
        raise KernelError(build.load().da_last_error().decode())


_VP, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_ARGTYPES = {
    "da_embed": [_VP, _VP, _VP, _I, _VP, _I, _VP, _I, _I, _F, _VP],
    "da_copy_rows": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _F, _VP],
    "da_take_tokens": [_VP, _VP, _VP, _I, _I, _I, _VP],
    "da_fill_zero": [_VP, ctypes.c_long, _VP],
    "da_state_gather": [_VP, _VP, _VP, _VP, _I, _I, _I, _VP],
    "da_state_scatter": [_VP, _VP, _VP, _VP, _I, _I, _I, _VP],
    "da_layernorm": [_VP, _VP, _VP, _I, _VP, _I, _F, _VP, _I, _I, _I, _VP],
    "da_gemm_ref": [_VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP],
    "da_gemm_bf16": [_VP, _I, _VP, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_gemm_bf16_wide": [_VP, _I, _VP, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP],
    "da_gemm_wide_choice": [_I, _I, _I],
    "da_gemm_bf16_ln": [_VP, _VP, _VP, _I, _VP, _I, _F, _VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP,
                        _I, _I, _I, _I, _I, _VP],
    "da_kv_write": [_VP, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _VP],
    "da_attn_ref": [_VP, _I, _VP, _I, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _VP],
    "da_attn_decode": [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _VP],
    "da_attn_decode_split": [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I, _VP, ctypes.c_long, _VP],
    "da_attn_prefill": [_VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I, _VP],
    "da_sample": [_VP, _I, _I, _I, _VP, _VP, _VP],
    "da_decode_splits": [_I, _I, _I, _I],
    "da_can_fuse_ln": [_I, _I, _I],
    "da_run_step": [_VP, _VP],
    "da_top_logprobs": [_VP, _I, _I, _I, _VP, _I, _VP, _VP, _VP],
}
_LIB = None


def _lib():
    """The kernel library with its argument types declared (conversion is then cheap and checked)."""
    global _LIB
    if _LIB is None:
        lib = build.load()
        for name, types in _ARGTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes = types
            fn.restype = ctypes.c_int
        _LIB = lib
    return _LIB


class _NoTiming:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_TIMING = _NoTiming()


def _timed(name: str, nbytes, flops, precision: str = "bf16"):
    """The kernel profiler's bracket around one launch, or nothing when it is off."""
    if not KernelProfiler.enabled:
        return _NO_TIMING
    return KernelProfiler.launch(name, nbytes, flops, precision)


def _nbytes(*ts) -> int:
    return sum(t.numel() * t.element_size() for t in ts if t is not None)


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")


def _rows_2d(t: torch.Tensor, name: str):
    if not (t.dim() == 2 and t.stride(1) == 1):
        raise KernelError(f"{name} must be 2-D with a contiguous last dimension")


# ------------------------------------------------------------------------------- embedding
def embed(tokens: torch.Tensor, positions: torch.Tensor, wte: torch.Tensor,
          wpe: Optional[torch.Tensor], out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[n] = wte[tokens[n]] * scale + wpe[positions[n]] in 32-bit."""
    _dev(tokens, positions, wte, wpe, out)
    N, E = out.shape
    _need(tokens.dtype == torch.int32 and positions.dtype == torch.int32, "embed: ids must be int32")
    _need(tokens.numel() >= N and positions.numel() >= N, "embed: fewer ids than rows")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
    _need(wte.is_contiguous() and wte.shape[1] == E, "embed: token table width differs from out")
    if wpe is not None:
        _need(wpe.is_contiguous() and wpe.shape[1] == E, "embed: position table width differs from out")
    with _timed("embed", N * E * (wte.element_size() * (2 if wpe is not None else 1) + 4), N * E, "fp32"):
        _check(_lib().da_embed(_ptr(tokens), _ptr(positions), _ptr(wte), _dt(wte), _ptr(wpe),
                               _dt(wpe) if wpe is not None else 0, _ptr(out), N, E, float(scale), _stream()))
    return out


def copy_rows(src: torch.Tensor, dst: torch.Tensor, rows: Optional[torch.Tensor] = None,
              accumulate: bool = False, scale: float = 1.0) -> torch.Tensor:
    """dst[r] (+)= scale * src[rows[r]] (or src[r]); 32-bit and bfloat16 on either side, += into 32-bit."""
    _dev(src, dst, rows)
    _need(src.dim() == 2 and dst.dim() == 2 and src.is_contiguous() and dst.is_contiguous() and
          src.shape[1] == dst.shape[1], "copy_rows: contiguous matrices of one width are needed")
    R = dst.shape[0]
    if rows is None:
        _need(src.shape[0] >= R, "copy_rows: fewer source rows than destination rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= R, "copy_rows: rows must be int32 with a row each")
    _need(not accumulate or dst.dtype == torch.float32, "copy_rows: accumulation needs a float32 destination")
    _check(_lib().da_copy_rows(_ptr(src), _dt(src), _ptr(rows), _ptr(dst), _dt(dst), R, dst.shape[1],
                               int(accumulate), float(scale), _stream()))
    return dst


def take_tokens(tokens: torch.Tensor, src: torch.Tensor, sampled: torch.Tensor, vocab: int) -> torch.Tensor:
    """tokens[n] = sampled[src[n]] wherever src[n] >= 0 (in place)."""
    _dev(tokens, src, sampled)
    _need(tokens.dtype == src.dtype == sampled.dtype == torch.int32, "take_tokens: int32 tensors needed")
    _need(src.numel() >= tokens.numel(), "take_tokens: fewer sources than tokens")
    _check(_lib().da_take_tokens(_ptr(tokens), _ptr(src), _ptr(sampled), tokens.numel(), sampled.numel(), int(vocab),
                                 _stream()))
    return tokens


def fill_zero(t: torch.Tensor) -> torch.Tensor:
    """Zeros over a contiguous tensor of whole 4-byte words, by a kernel of the engine's own (a recorded
    step then holds no memset node)."""
    _dev(t)
    _need(t.is_contiguous() and (t.numel() * t.element_size()) % 4 == 0, "fill_zero: a contiguous tensor of whole words")
    _check(_lib().da_fill_zero(_ptr(t), t.numel() * t.element_size(), _stream()))
    return t


def _state_rows(state: torch.Tensor, rows: torch.Tensor, name: str) -> int:
    _need(state.is_contiguous() and rows.is_contiguous() and state.dtype == rows.dtype and state.dim() >= 2,
          f"{name}: state [slots, ...] and rows [N, ...] must be contiguous and of one dtype")
    row_bytes = state[0].numel() * state.element_size()
    _need(rows.dim() >= 1 and rows.numel() == rows.shape[0] * state[0].numel() and row_bytes % 4 == 0,
          f"{name}: a row of the state is {state[0].numel()} entries ({row_bytes} bytes, whole words)")
    return row_bytes


def state_gather(state: torch.Tensor, state_slots: torch.Tensor, seq_of_token: torch.Tensor,
                 out: torch.Tensor) -> torch.Tensor:
    """out[n] = state[state_slots[seq_of_token[n]]]: every row of the step gets its sequence's state (zeros
    for a sequence without a slot, i.e. a padding row of a fixed-shape step)."""
    _dev(state, state_slots, seq_of_token, out)
    row_bytes = _state_rows(state, out, "state_gather")
    N = out.shape[0]
    _need(state_slots.dtype == torch.int32 and seq_of_token.dtype == torch.int32 and seq_of_token.numel() >= N,
          "state_gather: slots and sequence ids must be int32, one id a row")
    _check(_lib().da_state_gather(_ptr(state), _ptr(state_slots), _ptr(seq_of_token), _ptr(out), N, state.shape[0],
                                  row_bytes, _stream()))
    return out


def state_scatter(state: torch.Tensor, state_slots: torch.Tensor, q_start: torch.Tensor, rows: torch.Tensor,
                  n_seqs: int) -> None:
    """state[state_slots[s]] = rows[q_start[s + 1] - 1] for every sequence s with a slot: what the last row
    of a sequence's portion leaves is the request's state after the step."""
    _dev(state, state_slots, q_start, rows)
    row_bytes = _state_rows(state, rows, "state_scatter")
    _need(state_slots.dtype == torch.int32 and q_start.dtype == torch.int32 and state_slots.numel() >= n_seqs
          and q_start.numel() >= n_seqs + 1, "state_scatter: slots [S] and q_start [S+1] must be int32")
    _check(_lib().da_state_scatter(_ptr(state), _ptr(state_slots), _ptr(q_start), _ptr(rows), n_seqs, state.shape[0],
                                   row_bytes, _stream()))


# ------------------------------------------------------------------------------- norms
def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
              out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm of 32-bit rows; with ``rows`` the output row r is the norm of x[rows[r]]."""
    _dev(x, weight, bias, out, rows)
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2, "layernorm: x must be contiguous float32 [N, E]")
    E = x.shape[1]
    R = out.shape[0]
    _need(out.is_contiguous() and out.shape[1] == E, "layernorm: out must be contiguous [R, E]")
    _need(weight.numel() == E and (bias is None or bias.numel() == E), "layernorm: parameter length differs from E")
    if rows is None:
        _need(R <= x.shape[0], "layernorm: more output rows than input rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= R, "layernorm: rows must be int32 with R entries")
    with _timed("layernorm", R * E * (4 + out.element_size()) + _nbytes(weight, bias), 8 * R * E, "fp32"):
        _check(_lib().da_layernorm(_ptr(x), _ptr(rows), _ptr(weight), _dt(weight), _ptr(bias),
                                   _dt(bias) if bias is not None else 0, eps, _ptr(out),
                                   _dt(out), R, E, _stream()))
    return out


# ------------------------------------------------------------------------------- products
def linear_ref(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
               act: Optional[str] = None, accumulate: bool = False) -> torch.Tensor:
    """out (+)= act(a @ w.T + bias) with the plain tiled kernel; w is [N, K]."""
    _dev(a, w, bias, out)
    _rows_2d(a, "a"); _rows_2d(w, "w"); _rows_2d(out, "out")
    M, K = a.shape
    N = w.shape[0]
    if not (w.shape[1] == K):
        raise KernelError(f"linear: a is [{M},{K}] but w is {list(w.shape)}")
    if not (out.shape[0] == M and out.shape[1] == N):
        raise KernelError(f"linear: out is {list(out.shape)}, expected [{M},{N}]")
    _need(a.dtype == w.dtype, "linear: a and w must share a dtype")
    _need(bias is None or bias.numel() == N, "linear: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear: unknown activation {act!r}")
    _need(not accumulate or out.dtype == torch.float32, "linear: accumulation needs a float32 output")
    with _timed("linear_ref", _product_bytes(a, w, bias, out, accumulate), 2 * M * N * K, "fp32"):
        _check(_lib().da_gemm_ref(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _dt(a), _ptr(bias),
                                  _dt(bias) if bias is not None else 0, ACTIVATIONS[act], int(accumulate),
                                  _ptr(out), _dt(out), out.stride(0), M, N, K, _stream()))
    return out


def _product_bytes(a, w, bias, out, accumulate) -> int:
    """What a product must move at least: a, w and the bias once, the output once (twice when it adds)."""
    return _nbytes(a, w, bias) + _nbytes(out) * (2 if accumulate else 1)


# ------------------------------------------------------------------------------- cache write
def kv_write(qkv: torch.Tensor, k_off: int, v_off: int, cache_slot: torch.Tensor,
             slot_map: torch.Tensor, n_kv_heads: int, head_dim: int) -> None:
    """Rows of k and v (columns k_off.., v_off.. of qkv) go to cache rows ``slot_map``.
    cache_slot: [n_pages, 2, Hkv, page, D]."""
    _dev(qkv, cache_slot, slot_map)
    _rows_2d(qkv, "qkv")
    N = qkv.shape[0]
    _need(cache_slot.dim() == 5 and cache_slot.is_contiguous(), "kv_write: cache slot must be contiguous [pages,2,Hkv,page,D]")
    P, two, Hkv, page, D = cache_slot.shape
    _need(two == 2 and Hkv == n_kv_heads and D == head_dim, "kv_write: cache slot shape differs from the heads")
    _need(cache_slot.dtype == qkv.dtype, "kv_write: cache and activations differ in dtype")
    _need(slot_map.dtype == torch.int32 and slot_map.numel() >= N, "kv_write: slot_map must be int32 [N]")
    with _timed("kv_write", 4 * N * Hkv * D * qkv.element_size(), 0, "fp32"):
        _check(_lib().da_kv_write(_ptr(qkv), _dt(qkv), qkv.stride(0), k_off, v_off, _ptr(cache_slot),
                                  _ptr(slot_map), N, Hkv, D, page, _stream()))


# ------------------------------------------------------------------------------- attention
def attention_ref(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                  seq_of_token: torch.Tensor, positions: torch.Tensor, n_heads: int, scale: float,
                  window: Optional[int], out: torch.Tensor) -> torch.Tensor:
    """Plain paged attention for any rows.  q: [N, >= Hq*D] view (row stride free)."""
    _dev(q, cache_slot, block_table, seq_of_token, positions, out)
    _rows_2d(q, "q"); _rows_2d(out, "out")
    N = q.shape[0]
    P, two, Hkv, page, D = cache_slot.shape
    _need(cache_slot.is_contiguous() and two == 2, "attention: cache slot must be contiguous [pages,2,Hkv,page,D]")
    _need(q.shape[1] == n_heads * D and out.shape[1] == n_heads * D and out.shape[0] == N,
          "attention: q/out must be [N, Hq*D]")
    _need(q.dtype == cache_slot.dtype == out.dtype, "attention: q, cache and out must share a dtype")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention: block_table must be contiguous int32 [S, max_blocks]")
    _need(seq_of_token.dtype == torch.int32 and positions.dtype == torch.int32, "attention: ids must be int32")
    _need(seq_of_token.numel() >= N and positions.numel() >= N, "attention: fewer ids than rows")
    _check(_lib().da_attn_ref(_ptr(q), q.stride(0), _ptr(cache_slot), _dt(q), _ptr(block_table),
                              block_table.shape[1], _ptr(seq_of_token), _ptr(positions), N, n_heads, Hkv,
                              D, page, scale, int(window or 0), _ptr(out), out.stride(0),
                              _stream()))
    return out


# ------------------------------------------------------------------------------- sampling
SAMPLE_ROW_FLOATS = 8     # one SampleRow record is 8 four-byte fields


def sample(logits: torch.Tensor, params: torch.Tensor, out_tokens: torch.Tensor) -> torch.Tensor:
    """params: int32/float32-punned [R, 8] records (see sampling.device_rows)."""
    _dev(logits, params, out_tokens)
    _rows_2d(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "sample: logits must be float32")
    _need(params.is_contiguous() and params.numel() >= R * SAMPLE_ROW_FLOATS and params.element_size() == 4,
          "sample: params must hold R records of 8 four-byte fields")
    _need(out_tokens.dtype == torch.int32 and out_tokens.numel() >= R, "sample: out must be int32 [R]")
    with _timed("sample", R * V * 4, R * V, "fp32"):
        _check(_lib().da_sample(_ptr(logits), logits.stride(0), R, V, _ptr(params), _ptr(out_tokens), _stream()))
    return out_tokens


def top_logprobs(logits: torch.Tensor, params: torch.Tensor, n: int, out_idx: torch.Tensor,
                 out_lp: torch.Tensor) -> None:
    _dev(logits, params, out_idx, out_lp)
    _rows_2d(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "top_logprobs: logits must be float32")
    _need(0 < n <= V, "top_logprobs: n must be in [1, V]")
    _need(out_idx.dtype == torch.int32 and out_idx.numel() >= R * n and out_idx.is_contiguous(), "top_logprobs: out_idx")
    _need(out_lp.dtype == torch.float32 and out_lp.numel() >= R * n and out_lp.is_contiguous(), "top_logprobs: out_lp")
    _check(_lib().da_top_logprobs(_ptr(logits), logits.stride(0), R, V, _ptr(params), n, _ptr(out_idx),
                                        _ptr(out_lp), _stream()))


# ------------------------------------------------------------------------------- dispatch
# "tuned": MFMA products and the prefill/decode attention kernels in bfloat16;
# "reference": the plain kernels everywhere (for A/B checks).  32-bit always runs the plain
# kernels: they are its product path.
_MODE = "tuned"


def set_kernel_mode(mode: str) -> None:
    global _MODE
    if mode not in ("tuned", "reference"):
        raise ValueError("kernel mode must be 'tuned' or 'reference'")
    _MODE = mode


def kernel_mode() -> str:
    return _MODE


class kernel_mode_scope:
    """The kernel mode of one engine while one of its steps is put on the device (two engines of
    one process may differ)."""

    def __init__(self, mode: str):
        if mode not in ("tuned", "reference"):
            raise ValueError("kernel mode must be 'tuned' or 'reference'")
        self.mode = mode

    def __enter__(self):
        global _MODE
        self._old, _MODE = _MODE, self.mode
        return self

    def __exit__(self, *exc):
        global _MODE
        _MODE = self._old
        return False


def _kv_args(kv_cache, slot_map, q_cols, n_rows, N, out, name):
    """The cache-scatter arguments of a fused q|k|v projection (zeros when there is none)."""
    if kv_cache is None:
        return None, None, 0, 0, 0, 0, 0
    _need(kv_cache.dim() == 5 and kv_cache.is_contiguous() and kv_cache.dtype == torch.bfloat16 and
          out.dtype == torch.bfloat16, f"{name}: cache slot must be contiguous bfloat16 [pages,2,Hkv,page,D]")
    _, _, Hkv, page, D = kv_cache.shape
    _need(slot_map is not None and slot_map.dtype == torch.int32 and slot_map.numel() >= n_rows,
          f"{name}: slot_map must be int32 [rows]")
    if not (q_cols + 2 * Hkv * D == N):
        raise KernelError(f"{name}: q|k|v columns do not add up to N")
    return _ptr(kv_cache), _ptr(slot_map), q_cols, Hkv * D, Hkv, D, page


WIDE_TILE_SHAPES = {"wide": 0, "wide_256x128": 1, "wide_128x128": 2}


def _wide_tiles(M, N, K, act, accumulate, out) -> bool:
    """Whether the library gives this product to its tiles whose operands go straight into LDS (the
    profiler's name for it only; the choice itself is the library's: csrc/gemm_wide.hip)."""
    takes = K % 64 == 0 and (ACTIVATIONS[act] == 0 or (not accumulate and out.dtype == torch.bfloat16))
    return takes and _lib().da_gemm_wide_choice(M, N, K) >= 0


def linear_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                act: Optional[str] = None, accumulate: bool = False, kv_cache: Optional[torch.Tensor] = None,
                slot_map: Optional[torch.Tensor] = None, q_cols: int = 0, form: str = "auto") -> torch.Tensor:
    """out (+)= act(a @ w.T + bias) on the matrix cores; a, w bfloat16, K a multiple of 8.  With
    ``kv_cache`` the columns from ``q_cols`` on (k | v) also go to the cache rows ``slot_map``.
    ``form``: "auto" lets the library choose by shape; "wide", "wide_256x128" and "wide_128x128" ask for the
    tiles of 256 x 256, 256 x 128 and 128 x 128 whose operands go from memory straight into LDS, whatever
    the product's sizes (K a multiple of 64; tests and timing)."""
    _dev(a, w, bias, out)
    _rows_2d(a, "a"); _rows_2d(w, "w"); _rows_2d(out, "out")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "linear_mfma: a and w must be bfloat16")
    if not (w.shape[1] == K):
        raise KernelError(f"linear: a is [{M},{K}] but w is {list(w.shape)}")
    if not (out.shape[0] == M and out.shape[1] == N):
        raise KernelError(f"linear: out is {list(out.shape)}, expected [{M},{N}]")
    _need(bias is None or bias.numel() == N, "linear: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear: unknown activation {act!r}")
    _need(not accumulate or out.dtype == torch.float32, "linear: accumulation needs a float32 output")
    _need(kv_cache is None or not accumulate, "linear: a cache scatter goes with a plain store")
    kvp = _kv_args(kv_cache, slot_map, q_cols, M, N, out, "linear_mfma")
    timing = _NO_TIMING
    if KernelProfiler.enabled:           # (the cost model is worked out only when someone reads it)
        name = "product_skinny" if (M <= 32 or (M <= 64 and N <= 8192)) else ("product_wide" if _wide_tiles(M, N, K, act, accumulate, out) else "product_tile")
        timing = _timed(name, _product_bytes(a, w, bias, out, accumulate), 2 * M * N * K)
    if form != "auto" and form not in WIDE_TILE_SHAPES:
        raise KernelError(f"linear_mfma: unknown form {form!r}")
    args = (_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(bias), _dt(bias) if bias is not None else 0,
            ACTIVATIONS[act], int(accumulate), _ptr(out), _dt(out), out.stride(0), M, N, K, *kvp)
    with timing:
        if form == "auto":
            _check(_lib().da_gemm_bf16(*args, _stream()))
        else:
            _check(_lib().da_gemm_bf16_wide(*args, WIDE_TILE_SHAPES[form], _stream()))
    return out


# Which steps the fused norm + product kernel takes (few rows, a width it holds; measured limits) is the
# library's rule, da_can_fuse_ln in csrc/run_step.hip, so that the parts here and the step issued from C++
# decide alike.
FUSED_LN_KERNEL_MAX_ROWS = 32


def can_fuse_ln(n_rows: int, x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``linear_ln`` takes this step: few rows, bfloat16 weights, a width the kernel holds."""
    return (_MODE == "tuned" and w.dtype == torch.bfloat16 and x.dtype == torch.float32 and w.stride(0) % 8 == 0
            and bool(_lib().da_can_fuse_ln(int(n_rows), int(w.shape[1]), int(w.shape[0]))))


def linear_ln(x: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, norm_weight: torch.Tensor,
              norm_bias: Optional[torch.Tensor], eps: float, w: torch.Tensor, bias: Optional[torch.Tensor],
              out: torch.Tensor, act: Optional[str] = None, kv_cache: Optional[torch.Tensor] = None,
              slot_map: Optional[torch.Tensor] = None, q_cols: int = 0) -> torch.Tensor:
    """out = act(LayerNorm(x[rows]) @ w.T + bias) in one kernel, for steps of at most 32 rows; with
    ``kv_cache`` the columns from ``q_cols`` on (k | v of a fused projection) also go to the cache
    rows ``slot_map``."""
    _dev(x, rows, norm_weight, norm_bias, w, bias, out, kv_cache, slot_map)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "linear_ln: x must be contiguous float32")
    _rows_2d(w, "w"); _rows_2d(out, "out")
    N, K = w.shape
    _need(x.shape[1] == K and norm_weight.numel() == K and (norm_bias is None or norm_bias.numel() == K),
          "linear_ln: widths differ")
    _need(w.dtype == torch.bfloat16, "linear_ln: w must be bfloat16")
    _need(0 < n_rows <= FUSED_LN_KERNEL_MAX_ROWS and out.shape[0] >= n_rows and out.shape[1] == N, "linear_ln: bad row count")
    if rows is None:
        _need(x.shape[0] >= n_rows, "linear_ln: fewer rows in x than asked")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows, "linear_ln: rows must be int32")
    _need(bias is None or bias.numel() == N, "linear_ln: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear_ln: unknown activation {act!r}")
    kvp = _kv_args(kv_cache, slot_map, q_cols, n_rows, N, out, "linear_ln")
    with _timed("norm_product_fused", n_rows * K * 4 + _nbytes(w, bias, norm_weight, norm_bias) + n_rows * N * out.element_size(),
                2 * n_rows * N * K):
        _check(_lib().da_gemm_bf16_ln(
            _ptr(x), _ptr(rows), _ptr(norm_weight), _dt(norm_weight), _ptr(norm_bias),
            _dt(norm_bias) if norm_bias is not None else 0, eps, _ptr(w), w.stride(0), _ptr(bias),
            _dt(bias) if bias is not None else 0, ACTIVATIONS[act], _ptr(out), _dt(out), out.stride(0), n_rows, N, K,
            *kvp, _stream()))
    return out


def _mfma_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[1] % 8 == 0
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


# Measured on MI355X (q|k|v of 768 to 1,600 wide, 128 to 2,048 rows): the cache write in the product's
# epilogue adds 1.3 to 3.4 us where the rows' places are runs of consecutive cache rows (a prompt
# portion: keys and values both go over in 16-byte pieces), the write kernel after the product 3.7 to
# 9.2 us; with places in any order the two are level at 2,048 rows and the epilogue is ahead below.


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           act: Optional[str] = None, accumulate: bool = False, kv_cache: Optional[torch.Tensor] = None,
           slot_map: Optional[torch.Tensor] = None, q_cols: int = 0) -> torch.Tensor:
    """out (+)= act(a @ w.T + bias); picks the kernel by dtype and mode.  Shapes the matrix-core
    kernel does not take (K not a multiple of 8) go to the plain kernel, which takes any.  With
    ``kv_cache`` the k | v columns (from ``q_cols`` on) are also written to the cache rows
    ``slot_map``: in the product's epilogue on the matrix cores, by the write kernel otherwise."""
    if _MODE == "tuned" and _mfma_ok(a, w):
        return linear_mfma(a, w, bias, out, act, accumulate, kv_cache, slot_map, q_cols)
    linear_ref(a, w, bias, out, act, accumulate)
    if kv_cache is not None:
        _, _, Hkv, _, D = kv_cache.shape
        kv_write(out, q_cols, q_cols + Hkv * D, kv_cache, slot_map, Hkv, D)
    return out


def _attn_common(q, cache_slot, block_table, n_heads, out, name):
    _dev(q, cache_slot, block_table, out)
    _rows_2d(q, "q"); _rows_2d(out, "out")
    P, two, Hkv, page, D = cache_slot.shape
    if not (cache_slot.is_contiguous() and two == 2):
        raise KernelError(f"{name}: cache slot must be contiguous [pages,2,Hkv,page,D]")
    if not (q.shape[1] == n_heads * D and out.shape[1] == n_heads * D):
        raise KernelError(f"{name}: q/out must be [rows, Hq*D]")
    _need(q.dtype == torch.bfloat16 and cache_slot.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          f"{name}: q, cache and out must be bfloat16")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          f"{name}: block_table must be contiguous int32 [S, max_blocks]")
    return Hkv, page, D


def decode_splits(n_seqs: int, n_heads: int, max_blocks: int, page: int) -> int:
    """How many workgroups share a (sequence, head) pair's keys in decode attention (1: one workgroup a
    pair).  The library's rule (da_decode_splits in csrc/run_step.hip): from the step's shape only (pairs
    and the width of the block table), so that a recorded step keeps it."""
    return int(_lib().da_decode_splits(int(n_seqs), int(n_heads), int(max_blocks), int(page)))


def attention_decode(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                     seq_lens: torch.Tensor, n_seqs: int, n_heads: int, scale: float,
                     window: Optional[int], out: torch.Tensor, n_splits: int = 1,
                     workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One query row per sequence: row s of q belongs to sequence s and sits at position
    seq_lens[s] - 1.  With ``n_splits`` > 1 every (sequence, head) pair's keys are shared out over
    that many workgroups, whose partial results pass through ``workspace`` (float32,
    ``decode_workspace_floats`` elements)."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_decode")
    _need(q.shape[0] >= n_seqs and out.shape[0] >= n_seqs and block_table.shape[0] >= n_seqs,
          "attention_decode: fewer rows than sequences")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= n_seqs, "attention_decode: seq_lens must be int32 [S]")
    if n_splits <= 1:
        _check(_lib().da_attn_decode(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                     block_table.shape[1], _ptr(seq_lens), n_seqs, n_heads, Hkv, D, page,
                                     scale, int(window or 0), _ptr(out), out.stride(0), _stream()))
        return out
    need = decode_workspace_floats(n_seqs, n_heads, D, n_splits)
    _need(workspace is not None and workspace.dtype == torch.float32 and workspace.is_contiguous()
          and workspace.numel() >= need, f"attention_decode: the workspace must hold {need} float32")
    _dev(workspace)
    _check(_lib().da_attn_decode_split(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                       block_table.shape[1], _ptr(seq_lens), n_seqs, n_heads, Hkv, D, page,
                                       scale, int(window or 0), _ptr(out), out.stride(0), n_splits,
                                       _ptr(workspace), workspace.numel() * 4, _stream()))
    return out


def decode_workspace_floats(n_seqs: int, n_heads: int, head_dim: int, n_splits: int) -> int:
    return n_seqs * n_heads * n_splits * (head_dim + 2)


def attention_prefill(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                      q_start: torch.Tensor, seq_lens: torch.Tensor, seq0: int, n_seqs: int,
                      max_query_len: int, n_heads: int, scale: float, window: Optional[int],
                      out: torch.Tensor, form: int = 0) -> torch.Tensor:
    """Portions: sequence s (seq0 <= s < seq0 + n_seqs) owns rows q_start[s] .. q_start[s+1]-1 of q
    and out; its last row sits at position seq_lens[s] - 1.  ``form``: a workgroup's row blocks of 32 and
    the wavefronts that share out a row block's keys, as a two-digit number (41: any head size; 22: up to
    128; 42 and 14: up to 64); 0 lets the kernel choose from the step's shape."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_prefill")
    _need(q_start.dtype == torch.int32 and q_start.numel() >= seq0 + n_seqs + 1, "attention_prefill: q_start must be int32 [S+1]")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= seq0 + n_seqs, "attention_prefill: seq_lens must be int32 [S]")
    _need(block_table.shape[0] >= seq0 + n_seqs, "attention_prefill: block table has fewer rows than sequences")
    _need(q.shape[0] == out.shape[0], "attention_prefill: q and out differ in rows")
    _check(_lib().da_attn_prefill(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                        block_table.shape[1], _ptr(q_start), _ptr(seq_lens), seq0, n_seqs,
                                        max_query_len, n_heads, Hkv, D, page, scale,
                                        int(window or 0), _ptr(out), out.stride(0), form, _stream()))
    return out


def paged_attention(ctx, q: torch.Tensor, cache_slot: torch.Tensor, group: int, n_heads: int,
                    scale: float, window: Optional[int], out: torch.Tensor) -> torch.Tensor:
    """Attention of every row of the step over its sequence's pages.  In bfloat16 the one-token
    sequences (the first ``ctx.n_decode``) go to the decode kernel and the portions to the
    prefill kernel; 32-bit, the reference mode and head sizes that are no multiple of 16 (which the
    matrix-core kernels do not take) use the plain kernel for all rows."""
    bt = ctx.block_tables[group]
    Hkv, page, D = cache_slot.shape[2], cache_slot.shape[3], cache_slot.shape[4]
    el = cache_slot.element_size()
    nd = ctx.n_decode
    lens, starts = ctx.seq_lens_host, ctx.q_start_host        # for the profiler's cost model only

    def cost(first, last):
        """(bytes, flops) of the sequences first..last-1: every visible key and value once, q and out once;
        two products of 2 * D flops for every (query row, visible key, head)."""
        if not KernelProfiler.enabled or not lens:
            return 0, 0
        keys = pairs = rows = 0
        for s_ in range(first, last):
            t = starts[s_ + 1] - starts[s_]
            n = lens[s_]
            lo = 0 if not window else max(0, n - t - window + 1)
            keys += n - lo
            rows += t
            pairs += sum(min(n - t + i + 1, window or n) for i in range(t)) if t > 1 else min(n, window or n)
        return keys * 2 * Hkv * D * el + 2 * rows * n_heads * D * el, 4 * pairs * n_heads * D

    if _MODE == "tuned" and q.dtype == torch.bfloat16 and D % 16 == 0 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0:
        if nd:
            n_splits = decode_splits(nd, n_heads, bt.shape[1], page)
            ws = None
            if n_splits > 1:
                ws = ctx.buf("decode_partial", 1, decode_workspace_floats(nd, n_heads, D, n_splits), torch.float32)
            with _timed("attention_decode", *cost(0, nd)):
                attention_decode(q, cache_slot, bt, ctx.seq_lens, nd, n_heads, scale, window, out, n_splits, ws)
        if ctx.n_seqs > nd:
            with _timed("attention_prefill", *cost(nd, ctx.n_seqs)):
                attention_prefill(q, cache_slot, bt, ctx.q_start, ctx.seq_lens, nd, ctx.n_seqs - nd,
                                  ctx.max_query_len, n_heads, scale, window, out)
        return out
    with _timed("attention_plain", *cost(0, ctx.n_seqs), "fp32" if q.dtype == torch.float32 else "bf16"):
        return attention_ref(q, cache_slot, bt, ctx.seq_of_token, ctx.positions, n_heads, scale, window, out)
