"""Attention over a cached latent: the keys and values of all heads are products of one small vector a token."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import KVNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import build_part, register_part
from .spec import PartSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """``heads`` query heads of ``dim`` unrotated and ``rot_dim`` rotated elements (``q = W_q h``, head by head ``[dim | rot_dim]``).
    ``W_dkv h`` has ``kv_rank + rot_dim`` outputs: the first ``kv_rank``, RMS-normed with a gain, are the latent ``c``; the last
    ``rot_dim`` are one rotated key part that all heads share.  Head ``h``'s unrotated key is ``U_h c`` and its value ``V_h c``
    (the rows of ``W_uk`` and ``W_uv``, head by head); ``score = scale (q_u . k_u + q_r . k_r)``; causal; the softmax's
    denominator also holds ``exp(sink_h)`` (``sinks``); a head's result is multiplied by ``sigmoid(W_g h)_h``, one number a
    head (``gate``); output product.  The rotation turns neighbouring pairs of the rotated part (``position``: a part of a kind
    that rotates pairs over ``rot_dim`` elements).

    Only ``c`` and the rotated key part are cached, and the attention runs on them as they are: ``q_u . (U_h c) = (U_h^T q_u) .
    c`` and ``sum_j w_j V_h c_j = V_h sum_j w_j c_j``, so the cache entry is one key/value head with key rows ``[c | k_r]`` and
    value rows ``c``, the queries become ``[U_h^T q_u | q_r]`` (``ops.head_products``) and the heads' results go through
    ``V_h`` afterwards (the same kernel, with the gate).  Names: ``<prefix>q, dkv, dkv.norm, uk, uv, sink, g, o``."""

    def __init__(self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float, prefix: str,
                 eps: float = 1e-6, position: PartSpec | None = None, sinks: bool = True, gate: bool = True,
                 names: dict | None = None):
        if heads < 1 or dim < 0 or rot_dim < 0 or dim + rot_dim < 1 or vdim < 1 or kv_rank < 1:
            raise ConfigError(f"latent attention with {heads} heads of {dim} + {rot_dim}, values of {vdim}, latent {kv_rank}")
        if kv_rank + rot_dim > ops.GENERIC_MAX_HEAD_DIM:
            raise ConfigError(f"a latent of {kv_rank} + {rot_dim}: the attention kernel takes rows of up to {ops.GENERIC_MAX_HEAD_DIM}")
        self.hidden, self.heads, self.dim, self.rot, self.vdim, self.rank = hidden, heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.prefix, self.eps, self.sinks, self.gate = float(scale), prefix, eps, bool(sinks), bool(gate)
        self.position = build_part("position", position or PartSpec("none"))
        if position is not None and position.kind != "none" and not getattr(self.position, "pairs", False):
            raise ConfigError("the rotated part of a latent attention turns in neighbouring pairs")
        p = prefix
        self.names = {"q": p + "q", "dkv": p + "dkv", "c_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
                      "sink": p + "sink", "g": p + "g", "o": p + "o"}
        self.names.update(names or {})
        self.q_width = heads * (dim + rot_dim)

    def tensors(self):
        n, d = self.names, self.hidden
        t = {n["q"]: TensorSpec((self.q_width, d), MATRIX), n["dkv"]: TensorSpec((self.rank + self.rot, d), MATRIX),
             n["c_norm"]: TensorSpec((self.rank,), GAIN), n["uk"]: TensorSpec((self.heads * self.dim, self.rank), MATRIX),
             n["uv"]: TensorSpec((self.heads * self.vdim, self.rank), MATRIX),
             n["o"]: TensorSpec((d, self.heads * self.vdim), MATRIX)}
        if self.sinks:
            t[n["sink"]] = TensorSpec((self.heads,), GAIN)
        if self.gate:
            t[n["g"]] = TensorSpec((self.heads, d), MATRIX)
        t.update(self.position.tensors())
        return t

    def bind(self, weights, rt):
        self.rt = rt
        n = self.names
        rows = [weights[n["q"]], weights[n["dkv"]]] + ([weights[n["g"]]] if self.gate else [])
        self.w_in = rt.pack(rt.place_matrix(torch.cat(rows, 0)), always=True)       # q, the down projection and the gates in one
        self.c_gain = rt.place_gain(weights[n["c_norm"]])
        # per head: U_h^T as [dim, rank] (the rows of W_uk as they lie) and V_h^T as [rank, vdim]
        self.w_uk = rt.place_matrix(weights[n["uk"]]).view(self.heads, self.dim, self.rank).contiguous() if self.dim else None
        self.w_uv = rt.place_matrix(weights[n["uv"]]).view(self.heads, self.vdim, self.rank).transpose(1, 2).contiguous()
        self.sink = rt.place_gain(weights[n["sink"]]) if self.sinks else None
        self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)
        self.position.bind(weights, rt)
        table = self.position.rotation_table()
        turning = 0 if table is None else 2 * table.shape[0]
        if turning != self.rot:
            # the kernel rotates the whole rotated part: frequencies of 0 leave the pairs that do not turn as they are
            full = torch.zeros(self.rot // 2, dtype=torch.float32, device=rt.device)
            if table is not None:
                full[:table.shape[0]] = table
            table = full
        self.inv_freq = table if self.rot else None

    def cache_need(self):
        return KVNeed(1, self.rank + self.rot, None, self.rank)

    def forward(self, x, ctx, store, page_table):
        rt = self.rt
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_in))             # [T, q | c, k_r | g]
        kv_at = self.q_width
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            ops.latent_prepare(proj, 0, kv_at, self.c_gain, self.eps, self.inv_freq, ctx.tok_pos, ctx.tok_seq, page_table,
                               store.k_pages, store.v_pages, self.heads, self.dim, self.rot, self.rank)
            # steps of many bfloat16 tokens: the products per head as one batched product of the library
            batched = (not rt.invariant and proj.dtype == torch.bfloat16 and self.w_uv.dtype == torch.bfloat16
                       and proj.shape[0] >= ops.BATCHED_HEAD_PRODUCTS_FROM)
            if self.dim and batched:
                q = ops.head_products_batched(proj, 0, self.dim + self.rot, self.w_uk, self.heads, self.dim, self.rank,
                                              extra=self.rot)
            elif self.dim:
                q = ops.head_products(proj, 0, self.dim + self.rot, self.w_uk, self.heads, self.dim, self.rank, extra=self.rot)
            else:
                raise ConfigError("a latent attention without unrotated elements has no kernel")
        with profiler.section(profiler.ATTENTION):
            if not rt.invariant and ops.latent_attention_mfma_fits(q.dtype, self.rank + self.rot, self.rank, store.page_size):
                # the sizes the matrix cores take: a wavefront on 16 heads of a token walks the token's pages; a step of few
                # tokens cuts the pages into chunks side by side (one walk of 1,024 keys by the two wavefronts a sequence has
                # takes 319 us, the general kernel 106)
                o = ops.latent_attention_mfma(q, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, self.heads,
                                              self.scale, self.sink, ctx.max_len if ctx.is_decode else 0)
            else:
                o = ops.attention(q, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, self.heads, 1,
                                  self.rank + self.rot, None, self.scale, sinks=self.sink)
            if batched and o.dtype == torch.bfloat16:
                heads = ops.head_products_batched(o, 0, self.rank, self.w_uv, self.heads, self.rank, self.vdim,
                                                  gates=proj if self.gate else None, g_off=kv_at + self.rank + self.rot)
            else:
                heads = ops.head_products(o, 0, self.rank, self.w_uv, self.heads, self.rank, self.vdim,
                                          gates=proj if self.gate else None, g_off=kv_at + self.rank + self.rot)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(heads, self.w_o, out_dtype=torch.float32, parts_ok=True)
