"""A state-space mixer with a scalar decay per head: a state of fixed size and the tail of a short convolution per sequence."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import StateNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "state_space")
class StateSpaceMixer(Mixer):
    """The state-space duality form.  ``inner = heads * vdim``; ``W_in h`` is ``[z: inner | x: inner | B: groups * state | C: groups *
    state | dt: heads]``.  x, B and C together pass a causal convolution per channel (``taps`` taps, the last the current
    token's, zeros before a sequence's start, with a bias) and silu.  ``dt <- softplus(dt + dt_bias)`` without a clamp; per
    head ``h`` (which reads B and C of group ``h // (heads / groups)``)

        S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T,        y_t = S_t^T C_t + D_h x_t        (S is state x vdim).

    ``y``, heads side by side, is multiplied by ``silu(z)`` and then RMS-normed in ``norm_groups`` equal parts, each by its own
    root mean square, times a gain an element; output product.  The state and the convolution's last ``taps - 1`` inputs are
    float32 and live in the cache's state arenas at the sequence's slot.  Names: ``<prefix>in, conv, conv.b, dt_bias, A_log,
    D, norm, o``."""

    def __init__(self, hidden: int, heads: int, vdim: int, state: int, groups: int, taps: int, norm_groups: int, prefix: str,
                 eps: float = 1e-6, names: dict | None = None):
        if heads < 1 or groups < 1 or heads % groups or not 1 <= vdim <= 256 or not 1 <= state <= 1024:
            raise ConfigError(f"a state-space mixer with {heads} heads in {groups} groups, state {state} x {vdim}: the kernel "
                              "takes heads of up to 256 channels and states of up to 1,024 rows")
        if not 1 <= taps <= ops.SSD_MAX_TAPS:
            raise ConfigError(f"a convolution of {taps} taps: the kernel takes 1 to {ops.SSD_MAX_TAPS}")
        if norm_groups < 1 or (heads * vdim) % norm_groups:
            raise ConfigError(f"{heads * vdim} channels in {norm_groups} normed parts")
        self.hidden, self.heads, self.vdim, self.state, self.groups = hidden, heads, vdim, state, groups
        self.taps, self.norm_groups, self.prefix, self.eps = taps, norm_groups, prefix, eps
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state              # what the convolution runs over: x, B, C
        p = prefix
        self.names = {"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias",
                      "A_log": p + "A_log", "D": p + "D", "norm": p + "norm", "o": p + "o"}
        self.names.update(names or {})

    def tensors(self):
        n, d = self.names, self.hidden
        return {n["in"]: TensorSpec((self.inner + self.channels + self.heads, d), MATRIX),
                n["conv"]: TensorSpec((self.channels, self.taps), GAIN), n["conv_bias"]: TensorSpec((self.channels,), BIAS),
                n["dt_bias"]: TensorSpec((self.heads,), BIAS), n["A_log"]: TensorSpec((self.heads,), BIAS),
                n["D"]: TensorSpec((self.heads,), GAIN), n["norm"]: TensorSpec((self.inner,), GAIN),
                n["o"]: TensorSpec((d, self.inner), MATRIX)}

    def bind(self, weights, rt):
        self.rt = rt
        n = self.names
        self.w_in = rt.pack(rt.place_matrix(weights[n["in"]]), always=True)
        self.conv_w, self.conv_b = rt.place_gain(weights[n["conv"]]), rt.place_gain(weights[n["conv_bias"]])
        self.dt_bias, self.a_log = rt.place_gain(weights[n["dt_bias"]]), rt.place_gain(weights[n["A_log"]])
        self.d_skip, self.gain = rt.place_gain(weights[n["D"]]), rt.place_gain(weights[n["norm"]])
        self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)

    def cache_need(self):
        return (StateNeed((self.heads, self.state, self.vdim), torch.float32),
                StateNeed((max(self.taps - 1, 1), self.channels), torch.float32))

    def forward(self, x, ctx, store, page_table):
        rt = self.rt
        state, tails = store
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_in))             # [T, z | x, B, C | dt]
        with profiler.section(profiler.ATTENTION):
            xbc = ops.causal_conv_silu(proj, self.inner, self.channels, self.conv_w, self.conv_b, tails, ctx.tok_seq,
                                       ctx.cu_seqlens, ctx.slots)
            gn = self.groups * self.state
            y = ops.ssd_scan(xbc, self.inner, self.inner + gn, proj, 0, self.inner + self.channels, self.dt_bias, self.a_log,
                             self.d_skip, state, ctx.cu_seqlens, ctx.slots, self.heads, self.groups, self.state, self.vdim)
            y = ops.group_rms_norm(y, self.gain, self.eps, self.norm_groups, rt.dtype)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(y, self.w_o, out_dtype=torch.float32, parts_ok=True)
