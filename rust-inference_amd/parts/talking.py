"""Windowed attention whose values are its keys and whose heads talk after the softmax."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import KVNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, MATRIX, MIXING, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "talking_attention")
class TalkingAttention(Mixer):
    """``heads`` query heads over ``kv_heads`` key heads of ``dim`` (query head ``h`` reads key head ``h // (heads / kv_heads)``).
    ``q = W_q h``, ``k = W_k h``, and the values are the keys as projected: there is no value projection.  q and k are
    RMS-normed over the whole projection (all heads at once) with a gain an element; no rotation:
    ``score = scale (q . k) - r1_h ln(1 + r2_h (i - j))`` with two learned numbers a head (``distance_bias``); position ``i``
    sees ``j`` with ``0 <= i - j < window``; plain softmax; then the heads' weights are mixed, ``w'_h = sum_g T[h, g] w_g``
    (``talk``), and head ``h`` applies ``w'_h`` to the values of its own key head; the heads side by side are multiplied by
    ``sigmoid(W_g h)`` (``gate``) before the output product.  Names: ``<prefix>q, k, q.norm, k.norm, r1, r2, talk, g, o``.

    Beside other mixers (``parts.parallel.ParallelMixers``) it writes its gated heads into the row that the shared
    output product reads (``run_into``)."""

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, scale: float, prefix: str, eps: float = 1e-6,
                 window: int | None = None, distance_bias: bool = True, talk: bool = True, gate: bool = True,
                 names: dict | None = None):
        if heads < 1 or kv_heads < 1 or heads % kv_heads or dim < 1:
            raise ConfigError(f"{heads} attention heads over {kv_heads} key heads of {dim}")
        if heads * dim > 4096 or (heads * dim + 130 * heads) * 4 > 65536:
            raise ConfigError(f"{heads} talking heads of {dim}: the kernel takes up to 4,096 elements a token")
        if window is not None and window < 1:
            raise ConfigError(f"window {window} must be positive")
        self.hidden, self.heads, self.kv_heads, self.dim = hidden, heads, kv_heads, dim
        self.scale, self.prefix, self.eps, self.window = float(scale), prefix, eps, window
        self.distance_bias, self.talk, self.gate = bool(distance_bias), bool(talk), bool(gate)
        p = prefix
        self.names = {"q": p + "q", "k": p + "k", "q_norm": p + "q.norm", "k_norm": p + "k.norm", "r1": p + "r1", "r2": p + "r2",
                      "talk": p + "talk", "g": p + "g", "o": p + "o"}
        self.names.update(names or {})
        self.q_width, self.k_width = heads * dim, kv_heads * dim
        self.out_width = heads * dim

    def tensors(self):
        n, d = self.names, self.hidden
        t = {n["q"]: TensorSpec((self.q_width, d), MATRIX), n["k"]: TensorSpec((self.k_width, d), MATRIX),
             n["q_norm"]: TensorSpec((self.q_width,), GAIN), n["k_norm"]: TensorSpec((self.k_width,), GAIN),
             n["o"]: TensorSpec((d, self.out_width), MATRIX)}
        if self.distance_bias:
            t[n["r1"]] = TensorSpec((self.heads,), GAIN)
            t[n["r2"]] = TensorSpec((self.heads,), GAIN)
        if self.talk:
            t[n["talk"]] = TensorSpec((self.heads, self.heads), MIXING)
        if self.gate:
            t[n["g"]] = TensorSpec((self.out_width, d), MATRIX)
        return t

    def out_matrix(self, weights):
        return weights[self.names["o"]]

    def bind(self, weights, rt, alone: bool = True):
        self.rt = rt
        n = self.names
        rows = [weights[n["q"]], weights[n["k"]]] + ([weights[n["g"]]] if self.gate else [])
        self.w_in = rt.pack(rt.place_matrix(torch.cat(rows, 0)), always=True)
        if alone:
            self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)
        self.q_gain, self.k_gain = rt.place_gain(weights[n["q_norm"]]), rt.place_gain(weights[n["k_norm"]])
        self.r1 = rt.place_gain(weights[n["r1"]]) if self.distance_bias else None
        self.r2 = rt.place_gain(weights[n["r2"]]) if self.distance_bias else None
        self.mix = rt.place_gain(weights[n["talk"]]) if self.talk else None

    def cache_need(self):
        return KVNeed(self.kv_heads, self.dim, self.window)

    def run_into(self, x, ctx, store, page_table, out, out_col: int, out_scale: float, residual=None) -> None:
        """The mixer up to its output product: the gated heads, times ``out_scale``, into the columns ``out_col ..`` of ``out``."""
        rt = self.rt
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_in))             # [T, q | k | g]
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            ops.whole_norm_kv_write(proj, 0, self.q_width, self.q_gain, self.k_gain, self.eps, ctx.tok_pos, ctx.tok_seq,
                                    page_table, store.k_pages, store.v_pages, self.heads, self.kv_heads, self.dim)
        with profiler.section(profiler.ATTENTION):
            # a step of few tokens cuts its walk over the keys into shares that run side by side
            longest = min(ctx.max_len, self.window) if self.window else ctx.max_len
            shares = 1 if rt.dtype == torch.float32 or rt.invariant else ops.talking_attention_shares(proj.shape[0], longest)
            if (not ctx.is_decode and not rt.invariant and proj.shape[1] % 8 == 0
                    and ops.talking_attention_mfma_fits(proj.dtype, self.heads, self.kv_heads, self.dim, store.page_size)):
                # prompts at the sizes the matrix cores take: tiles of 16 tokens, both walks on them
                o = ops.talking_attention_mfma(proj, 0, store.k_pages, store.v_pages, ctx.tok_pos, ctx.cu_seqlens, ctx.new_counts,
                                               page_table, self.heads, self.kv_heads, self.dim, self.window, self.scale, self.r1,
                                               self.r2, self.mix)
            else:
                o = ops.talking_attention(proj, 0, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, self.heads,
                                          self.kv_heads, self.dim, self.window, self.scale, self.r1, self.r2, self.mix, shares)
            ops.gate_rows(out, out_col, o, proj if self.gate else None, self.q_width + self.k_width, out_scale, ops.GATE_SIGMOID)

    def forward(self, x, ctx, store, page_table):
        heads = torch.empty((x.shape[0], self.out_width), dtype=self.rt.dtype, device=self.rt.device)
        self.run_into(x, ctx, store, page_table, heads, 0, 1.0)
        with profiler.section(profiler.OUT_PROJECTION):
            return self.rt.linear_packed(heads, self.w_o, out_dtype=torch.float32, parts_ok=True)
