"""Time mixing with a decay per channel: a mixer that keeps a state of fixed size and its last input per sequence."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import StateNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "time_mix")
class TimeMix(Mixer):
    """With ``h'`` the input of the token before (zeros for a sequence's first token), each of r, k, v, g and w reads its own
    mix ``h + (h' - h) mu_s``.  ``r, k, v = W_r, W_k, W_v`` of their mixes (``heads x dim``), ``gate = silu(W_g mix_g)``, and the
    decay ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))`` per head and key channel (a product through a narrow middle whose
    width the checkpoint gives).  Per head

        o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,        S_t = diag(w_t) S_(t-1) + k_t v_t^T,

    the bonus ``u`` for the current token alone.  Each head's ``o`` is divided by its root mean square, the heads side by
    side are multiplied by a gain an element and by the gate, then the output product.  The state ``[heads, dim, dim]`` and
    the last input ``[hidden]`` are float32 and live in the cache's state arenas at the sequence's slot; the mixes are made
    from the float32 residual where the layer hands it over (``wants_residual``), so what is kept of the input is not
    rounded.  Names: ``<prefix>mu.r, mu.k, mu.v, mu.g, mu.w, r, k, v, g, w1, w2, w0, u, norm, o``."""

    wants_residual = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden: int, heads: int, dim: int, prefix: str, eps: float = 1e-6, decay_rank: int | None = None,
                 names: dict | None = None):
        if heads < 1 or not 1 <= dim <= ops.timemix_max_dim():
            raise ConfigError(f"time mixing with {heads} heads of {dim}: the kernel takes heads of 1 to {ops.timemix_max_dim()}")
        self.hidden, self.heads, self.dim, self.prefix, self.eps, self.decay_rank = hidden, heads, dim, prefix, eps, decay_rank
        p = prefix
        self.names = {"r": p + "r", "k": p + "k", "v": p + "v", "g": p + "g", "w1": p + "w1", "w2": p + "w2", "w0": p + "w0",
                      "u": p + "u", "norm": p + "norm", "o": p + "o"}
        self.names.update({"mu_" + s: p + "mu." + s for s in self.MIXES})
        self.names.update(names or {})
        self.width = self.out_width = heads * dim

    def tensors(self):
        n, d, w = self.names, self.hidden, self.width
        t = {n["mu_" + s]: TensorSpec((d,), GAIN) for s in self.MIXES}
        t.update({n[x]: TensorSpec((w, d), MATRIX) for x in ("r", "k", "v", "g")})
        t.update({n["w1"]: TensorSpec((self.decay_rank, d), MATRIX), n["w2"]: TensorSpec((w, self.decay_rank), MATRIX),
                  n["w0"]: TensorSpec((w,), BIAS), n["u"]: TensorSpec((self.heads, self.dim), GAIN),
                  n["norm"]: TensorSpec((w,), GAIN), n["o"]: TensorSpec((d, w), MATRIX)})
        return t

    def out_matrix(self, weights):
        return weights[self.names["o"]]

    def bind(self, weights, rt, alone: bool = True):
        self.rt = rt
        n = self.names
        if weights[n["w1"]].shape[0] != weights[n["w2"]].shape[1]:
            raise ConfigError(f"{n['w1']} has {weights[n['w1']].shape[0]} rows, {n['w2']} {weights[n['w2']].shape[1]} columns")
        self.mu = torch.stack([rt.place_gain(weights[n["mu_" + s]]) for s in self.MIXES], 0).contiguous()
        self.w = {x: rt.pack(rt.place_matrix(weights[n[x]])) for x in ("r", "k", "v", "g", "w1", "w2")}
        self.w0, self.u = rt.place_gain(weights[n["w0"]]), rt.place_gain(weights[n["u"]]).reshape(-1).contiguous()
        self.gain = rt.place_gain(weights[n["norm"]])
        if alone:
            self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)

    def cache_need(self):
        return (StateNeed((self.heads, self.dim, self.dim), torch.float32), StateNeed((self.hidden,), torch.float32))

    def run_into(self, x, ctx, store, page_table, out, out_col: int, out_scale: float, residual=None) -> None:
        """The mixer up to its output product: the normed and gated heads, times ``out_scale``, into the columns
        ``out_col ..`` of ``out``."""
        rt = self.rt
        state, kept = store
        x32 = residual if residual is not None else ops.as_rows(x).to(torch.float32)
        with profiler.section(profiler.QKV_PROJECTION):
            mixes = ops.shift_mix(x32, kept, self.mu, ctx.tok_seq, ctx.cu_seqlens, ctx.slots, rt.dtype)
            ops.shift_keep(kept, x32, ctx.cu_seqlens, ctx.slots)
            r, k, v, g = (ops.as_rows(rt.linear_packed(mixes[i], self.w[s])) for i, s in enumerate(("r", "k", "v", "g")))
            # the decay's pre-activation: tanh in float32 between its two products, the second one's sums float32
            mid = ops.tanh_rows(ops.as_rows(rt.linear_packed(mixes[4], self.w["w1"], out_dtype=torch.float32)), rt.dtype)
            z = ops.as_rows(rt.linear_packed(mid, self.w["w2"], out_dtype=torch.float32))
        with profiler.section(profiler.ATTENTION):
            ops.timemix_scan(out, out_col, out_scale, r, k, v, g, z, self.w0, self.u, self.gain, self.eps, state,
                             ctx.cu_seqlens, ctx.slots, self.heads, self.dim)

    def forward(self, x, ctx, store, page_table, residual=None):
        heads = torch.empty((x.shape[0], self.out_width), dtype=self.rt.dtype, device=self.rt.device)
        self.run_into(x, ctx, store, page_table, heads, 0, 1.0, residual)
        with profiler.section(profiler.OUT_PROJECTION):
            return self.rt.linear_packed(heads, self.w_o, out_dtype=torch.float32, parts_ok=True)
