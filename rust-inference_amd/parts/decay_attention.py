"""Linear attention with a fixed decay per head: a state of fixed size per sequence, no keys and values kept."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import StateNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "decay_attention")
class DecayLinearAttention(Mixer):
    """Per head, with ``q = silu(W_q h)``, ``k = silu(W_k h)`` (``heads x dim``), ``v = silu(W_v h)`` (``heads x vdim``) and
    one constant ``decay`` per head (a parameter, not a tensor):

        S_t = decay_h S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t        (no other scale).

    The heads side by side go through one RMS norm over all of them together (a gain of ``heads * vdim``), are
    multiplied by ``sigmoid(W_g h)`` and projected by ``W_o``.  The state ``[heads, dim, vdim]`` starts at zero and is
    float32, as are the decays, the activations on their way into the recurrence and its sums; it lives in the
    cache's state arena at the sequence's slot, so a sequence goes on from it in any later step.

    ``names``: checkpoint names of ``q, k, v, g, o, norm`` where they are not ``<prefix>q`` and so on.  The mixer can
    run beside another one on one input and one output product (``parts.parallel.ParallelMixers``):
    ``in_matrix``, ``core`` and ``out_matrix`` are its three steps taken apart.
    """

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, decay: tuple, prefix: str, eps: float = 1e-5,
                 gate: str | None = "sigmoid", names: dict | None = None):
        if heads < 1 or not 1 <= dim <= ops.GLA_MAX_DIM or vdim < 1:
            raise ConfigError(f"linear attention with {heads} heads of {dim} x {vdim}: the kernel takes key heads of 1 to "
                              f"{ops.GLA_MAX_DIM}")
        if len(decay) != heads:
            raise ConfigError(f"{len(decay)} decays for {heads} heads")
        if gate not in (None, "sigmoid", "silu"):
            raise ConfigError(f"an output gate {gate!r} is neither 'sigmoid' nor 'silu'")
        self.hidden, self.heads, self.dim, self.vdim = hidden, heads, dim, vdim
        self.decay, self.prefix, self.eps, self.gate = tuple(float(d) for d in decay), prefix, eps, gate
        p = prefix
        self.names = {"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "o": p + "o", "norm": p + "norm"}
        self.names.update(names or {})
        self.qk_width, self.out_width = heads * dim, heads * vdim
        self.in_width = 2 * self.qk_width + self.out_width * (2 if gate else 1)

    def tensors(self):
        n, d, hk, hv = self.names, self.hidden, self.qk_width, self.out_width
        t = {n["q"]: TensorSpec((hk, d), MATRIX), n["k"]: TensorSpec((hk, d), MATRIX), n["v"]: TensorSpec((hv, d), MATRIX),
             n["o"]: TensorSpec((d, hv), MATRIX), n["norm"]: TensorSpec((hv,), GAIN)}
        if self.gate:
            t[n["g"]] = TensorSpec((hv, d), MATRIX)
        return t

    def in_matrix(self, weights):
        n = self.names
        return torch.cat([weights[n[x]] for x in (("q", "k", "v", "g") if self.gate else ("q", "k", "v"))], 0)

    def out_matrix(self, weights):
        return weights[self.names["o"]]

    def bind(self, weights, rt, alone: bool = True):
        self.rt = rt
        if alone:
            self.w_in = rt.pack(rt.place_matrix(self.in_matrix(weights)), always=True)
            self.w_o = rt.pack(rt.place_matrix(weights[self.names["o"]]), parts_ok=True)
        self.gain = rt.place_gain(weights[self.names["norm"]])
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=rt.device)
        self.step_fits = ops.gla_step_fits(self.dim, self.vdim)

    def cache_need(self):
        return StateNeed((self.heads, self.dim, self.vdim), torch.float32)

    def core(self, proj, col0: int, ctx, store, page_table, out, out_col: int, out_scale: float) -> None:
        """``proj [T, row]`` holds this mixer's q, k, v (and g) from column ``col0`` on; the normed and gated heads,
        times ``out_scale``, are written into the columns ``out_col ..`` of ``out``."""
        hk, hv = self.qk_width, self.out_width
        with profiler.section(profiler.ATTENTION):
            if ctx.is_decode and self.step_fits and not self.rt.invariant:
                # one new token a sequence: the state in 16-byte pieces, a workgroup a sequence and head
                o = ops.decay_step(proj, col0, col0 + hk, col0 + 2 * hk, self.head_decay, 1.0, store, ctx.slots, self.heads,
                                   self.dim, self.vdim)
            elif (proj.dtype != torch.float32 and not self.rt.invariant
                  and ops.decay_chunks_pay(ctx.B, proj.shape[0], ctx.max_new, self.heads, self.dim, self.vdim)
                  and ops.decay_chunks_fit(self.dim, self.vdim, proj.shape[1], (col0, col0 + hk, col0 + 2 * hk))):
                # prompts: chunks of 64 tokens side by side instead of a walk token by token
                # (float32 and the invariant mode keep the one form of the walk)
                o = ops.decay_scan_chunked(proj, col0, col0 + hk, col0 + 2 * hk, self.head_decay, 1.0, store, ctx.cu_seqlens,
                                           ctx.slots, self.heads, self.dim, self.vdim, ctx.max_new)
            else:
                o = ops.decay_scan(proj, col0, col0 + hk, col0 + 2 * hk, self.head_decay, 1.0, store, ctx.cu_seqlens,
                                   ctx.slots, self.heads, self.dim, self.vdim)
            ops.row_norm_gate(out, out_col, o, self.gain, self.eps, proj if self.gate else None, col0 + 2 * hk + hv, out_scale,
                              ops.GATE_SILU if self.gate == "silu" else ops.GATE_SIGMOID)

    def forward(self, x, ctx, store, page_table):
        rt = self.rt
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_in))
        heads = torch.empty((proj.shape[0], self.out_width), dtype=proj.dtype, device=proj.device)
        self.core(proj, 0, ctx, store, page_table, heads, 0, 1.0)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(heads, self.w_o, out_dtype=torch.float32, parts_ok=True)
