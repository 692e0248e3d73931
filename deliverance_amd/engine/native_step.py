"""The step's forward pass issued from C++ in one call (``da_run_step``, csrc/run_step.h).

A model whose parts are all of the standard kinds (LayerNorm in front of each part, attention
without a rotation of q and k, a dense feed-forward or none, learned or no positions, bfloat16
weights) is described once as a record per entry of the run order; a step then fills one record
with its sizes, the addresses of its integer arrays and scratch buffers, and the library walks the
layers.  The kernels and their arguments are those that the parts launch one by one, so both ways
give the same bits; what the plan cannot describe (other parts, the 32-bit path, the plain kernels,
the debug hook, the kernel profiler) keeps going through the parts.
Reference: the layer loop of core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:1097-1118.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..kernels import ops
from ..parts.attention import CausalSelfAttention
from ..parts.feedforward import DenseFeedForward
from ..parts.norms import LayerNorm
from ..parts.positions import LearnedPositions, NoPositions

MAX_GROUPS = 4
_VP, _I, _F, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long


class DaNorm(ctypes.Structure):
    _fields_ = [("weight", _VP), ("bias", _VP), ("weight_dtype", _I), ("bias_dtype", _I), ("eps", _F), ("pad_", _I)]


class DaCall(ctypes.Structure):
    _fields_ = [("norm1", DaNorm), ("norm2", DaNorm),
                ("qkv_w", _VP), ("qkv_b", _VP), ("out_w", _VP), ("out_b", _VP), ("qkv_b_dtype", _I), ("out_b_dtype", _I),
                ("n_heads", _I), ("n_kv_heads", _I), ("head_dim", _I), ("window", _I), ("scale", _F), ("write", _I),
                ("kv_cache", _VP), ("group", _I), ("has_ff", _I),
                ("fc_w", _VP), ("fc_b", _VP), ("proj_w", _VP), ("proj_b", _VP), ("fc_b_dtype", _I), ("proj_b_dtype", _I),
                ("inner", _I), ("act", _I)]


class DaModel(ctypes.Structure):
    _fields_ = [("width", _I), ("vocab", _I), ("n_calls", _I), ("page", _I),
                ("token_table", _VP), ("pos_table", _VP), ("token_dtype", _I), ("pos_dtype", _I),
                ("embed_scale", _F), ("pad_", _I), ("final_norm", DaNorm), ("head_w", _VP), ("calls", ctypes.POINTER(DaCall))]


class DaStep(ctypes.Structure):
    _fields_ = [("N", _I), ("S", _I), ("n_decode", _I), ("R", _I), ("max_query_len", _I), ("n_groups", _I),
                ("tokens", _VP), ("positions", _VP), ("seq_of_token", _VP), ("q_start", _VP), ("seq_lens", _VP),
                ("want_rows", _VP), ("slot_map", _VP * MAX_GROUPS), ("block_table", _VP * MAX_GROUPS),
                ("max_blocks", _I * MAX_GROUPS),
                ("residual", _VP), ("norm", _VP), ("qkv", _VP), ("attn_out", _VP), ("ff_mid", _VP), ("final_norm", _VP),
                ("logits", _VP), ("decode_partial", _VP), ("decode_partial_floats", _L), ("stream", _VP)]


def _dt(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else ops._dt(t)


def _norm_record(norm: LayerNorm) -> DaNorm:
    return DaNorm(norm.weight.data_ptr(), None if norm.bias is None else norm.bias.data_ptr(), _dt(norm.weight),
                  _dt(norm.bias), norm.eps, 0)


class NativeStep:
    """The plan of one model on one cache, and the call that runs a step through it."""

    def __init__(self, model, cache):
        self.model = model
        self.cache = cache
        cfg = model.config
        n = len(cfg.schedule)
        self._calls = (DaCall * n)()
        self.qkv_cols = self.q_cols = self.inner = 0
        self._decode_shapes = []                      # (heads, head size, group) of every call, for the decode scratch
        for i, call in enumerate(cfg.schedule):
            blk = model.blocks[call.layer]
            at, ff = blk.mixer, blk.feed_forward
            rec = self._calls[i]
            rec.norm1 = _norm_record(blk.pre_mixer_norm)
            rec.qkv_w, rec.qkv_b = at.qkv_weight.data_ptr(), None if at.qkv_bias is None else at.qkv_bias.data_ptr()
            rec.out_w, rec.out_b = at.out_weight.data_ptr(), None if at.out_bias is None else at.out_bias.data_ptr()
            rec.qkv_b_dtype, rec.out_b_dtype = _dt(at.qkv_bias), _dt(at.out_bias)
            rec.n_heads, rec.n_kv_heads, rec.head_dim = at.n_heads, at.n_kv_heads, at.head_dim
            rec.window, rec.scale, rec.write = int(at.window or 0), at.scale, int(bool(call.write))
            rec.kv_cache, rec.group = cache.kv[call.cache].data_ptr(), cache.group_of_slot[call.cache]
            rec.has_ff = int(ff is not None)
            if ff is not None:
                rec.norm2 = _norm_record(blk.pre_ff_norm)
                rec.fc_w, rec.fc_b = ff.fc_weight.data_ptr(), None if ff.fc_bias is None else ff.fc_bias.data_ptr()
                rec.proj_w, rec.proj_b = ff.proj_weight.data_ptr(), None if ff.proj_bias is None else ff.proj_bias.data_ptr()
                rec.fc_b_dtype, rec.proj_b_dtype = _dt(ff.fc_bias), _dt(ff.proj_bias)
                rec.inner, rec.act = ff.inner, ops.ACTIVATIONS[ff.activation]
                self.inner = max(self.inner, ff.inner)
            self.qkv_cols, self.q_cols = max(self.qkv_cols, at.qkv_cols), max(self.q_cols, at.q_cols)
            self._decode_shapes.append((at.n_heads, at.head_dim, rec.group))
        pos = model.embed_position.embed_table()
        self._model = DaModel(cfg.width, cfg.vocab_size, n, cache.page_size, model.token_table.data_ptr(),
                              None if pos is None else pos.data_ptr(), _dt(model.token_table), _dt(pos), float(cfg.embed_scale), 0,
                              _norm_record(model.final_norm), model.head_weight.data_ptr(), self._calls)
        self._step = DaStep()
        self._run = ops._lib().da_run_step
        self._partial_floats = {}                     # (one-token sequences, block-table widths) -> floats of decode scratch

    @staticmethod
    def takes(model, cache, kernels: str) -> bool:
        """Whether every part of the model is one the plan describes (exact classes: a subclass may do
        anything in its ``forward``)."""
        if kernels != "tuned" or model.dtype != torch.bfloat16 or len(cache.groups) > MAX_GROUPS:
            return False
        if model.device.type != "cuda":
            return False
        cfg = model.config
        if cfg.width % 8 or type(model.final_norm) is not LayerNorm or model.head_weight.dtype != torch.bfloat16 or cfg.logit_multiplier != 1.0:
            return False
        if type(model.embed_position) not in (LearnedPositions, NoPositions):
            return False
        for blk in model.blocks:
            at, ff = blk.mixer, blk.feed_forward
            if type(at) is not CausalSelfAttention or at.position is not None or at.head_dim % 16 or at.head_dim > 256:
                return False
            if (type(blk.pre_mixer_norm) is not LayerNorm or blk.post_mixer_norm is not None or blk.post_ff_norm is not None
                    or blk.post_block_norm is not None or blk.residual_multiplier != 1.0):
                return False
            if ff is not None and (type(ff) is not DenseFeedForward or type(blk.pre_ff_norm) is not LayerNorm or ff.inner % 8):
                return False
        return True

    def forward(self, ctx, want_rows: Optional[torch.Tensor], n_want: int) -> torch.Tensor:
        """What ``CausalLM.forward`` returns for this step: logits [n_want, V] of the wanted rows."""
        N, cfg = ctx.n_tokens, self.model.config
        bf = torch.bfloat16
        st = self._step
        st.N, st.S, st.n_decode, st.R, st.max_query_len = N, ctx.n_seqs, ctx.n_decode, n_want, ctx.max_query_len
        st.n_groups = len(ctx.block_tables)
        st.tokens, st.positions, st.seq_of_token = ctx.tokens.data_ptr(), ctx.positions.data_ptr(), ctx.seq_of_token.data_ptr()
        st.q_start, st.seq_lens = ctx.q_start.data_ptr(), ctx.seq_lens.data_ptr()
        st.want_rows = want_rows.data_ptr() if n_want else None
        for g, (bt, sm) in enumerate(zip(ctx.block_tables, ctx.slot_maps)):
            st.slot_map[g], st.block_table[g], st.max_blocks[g] = sm.data_ptr(), bt.data_ptr(), bt.shape[1]
        # the same scratch buffers, under the same names, as the parts ask for
        st.residual = ctx.buf("residual", N, cfg.width, torch.float32).data_ptr()
        st.norm = ctx.buf("norm", N, cfg.width, bf).data_ptr()
        st.qkv = ctx.buf("qkv", N, self.qkv_cols, bf).data_ptr()
        st.attn_out = ctx.buf("attn_out", N, self.q_cols, bf).data_ptr()
        st.ff_mid = ctx.buf("ff_mid", N, self.inner, bf).data_ptr() if self.inner else None
        logits = ctx.buf("logits", n_want, cfg.vocab_size, torch.float32)
        st.logits = logits.data_ptr()
        st.final_norm = ctx.buf("final_norm", n_want, cfg.width, bf).data_ptr() if n_want else None
        floats = 0
        if ctx.n_decode:
            key = (ctx.n_decode, tuple(bt.shape[1] for bt in ctx.block_tables))
            floats = self._partial_floats.get(key)
            if floats is None:
                floats = 0
                for heads, d, g in self._decode_shapes:
                    splits = ops.decode_splits(ctx.n_decode, heads, key[1][g], self.cache.page_size)
                    if splits > 1:
                        floats = max(floats, ops.decode_workspace_floats(ctx.n_decode, heads, d, splits))
                self._partial_floats[key] = floats
        st.decode_partial = ctx.buf("decode_partial", 1, floats, torch.float32).data_ptr() if floats else None
        st.decode_partial_floats = floats
        st.stream = ops._stream()
        if self._run(ctypes.byref(self._model), ctypes.byref(st)) != 0:
            raise ops.KernelError(ops._lib().da_last_error().decode())
        return logits
