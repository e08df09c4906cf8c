"""Position encodings."""
from __future__ import annotations

import torch

from ..errors import ConfigError
from .base import PositionEncoding
from .registry import register_part


@register_part("position", "rotate_half")
class RotateHalf(PositionEncoding):
    """Rotary encoding of the "default" kind over the whole head, pairs ``(d, d + dh/2)``.
    ``inv_freq[i] = 1 / theta^(2i / dh)`` in float32 (the reference: src/ops/rope.rs:20);
    the kernel forms the angle ``f32(pos) * inv_freq[i]`` in float32 (:39) and rotates
    ``x'[d] = x[d] cos - x[d+half] sin``, ``x'[d+half] = x[d+half] cos + x[d] sin`` (:73-74)."""

    def __init__(self, head_dim: int, theta: float):
        if head_dim % 2:
            raise ConfigError(f"head_dim {head_dim} must be even for a rotation in pairs")
        self.head_dim, self.theta = head_dim, theta

    def bind(self, weights, rt):
        self.rt = rt
        i = torch.arange(self.head_dim // 2, dtype=torch.float32)
        expo = (2.0 * i) / torch.tensor(float(self.head_dim), dtype=torch.float32)
        theta = torch.tensor(self.theta, dtype=torch.float32)
        self.inv_freq = (1.0 / torch.pow(theta, expo)).to(torch.float32).to(rt.device).contiguous()

    def bind_plain(self, weights):
        from ..kernels import plain
        self.inv_freq_plain = plain.rope_inv_freq(self.head_dim, self.theta)

    def plain(self, heads, positions):
        """Rotates ``heads: [tokens, n, head_dim]`` (already normed) by their tokens' positions."""
        from ..kernels import plain
        return plain.rope(heads, positions, self.inv_freq_plain)

    def rotation_table(self):
        return self.inv_freq


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position enters the mixer (order then comes from the causal mask alone)."""

    def __init__(self, **_):
        pass

    def bind_plain(self, weights):
        pass

    def plain(self, heads, positions):
        return heads


@register_part("position", "rotate_pairs")
class RotatePairs(PositionEncoding):
    """Rotary encoding over the first ``dims`` elements of a head, in neighbouring pairs: the elements ``(2i, 2i + 1)``
    at position ``p`` turn by the angle ``p * base^(-2i / dims)`` (``i < dims / 2``); what lies behind ``dims`` passes
    unchanged.  The frequencies are rounded to float32 once; angle, sine and cosine are float32 in the kernel.
    ``pairs`` tells the mixer that neighbours turn (not the halves of a head): it then rotates before it norms."""

    pairs = True

    def __init__(self, head_dim: int, dims: int, base: float):
        if dims % 2 or not 0 <= dims <= head_dim:
            raise ConfigError(f"a rotation over {dims} of {head_dim} elements: an even number up to the head size")
        if dims and not base > 0:
            raise ConfigError(f"the rotation's base {base} must be positive")
        self.head_dim, self.dims, self.base = head_dim, dims, float(base)

    def bind(self, weights, rt):
        self.rt = rt
        self.inv_freq = None
        if self.dims:
            i = torch.arange(self.dims // 2, dtype=torch.float64)
            self.inv_freq = torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / self.dims) \
                .to(torch.float32).to(rt.device).contiguous()

    def rotation_table(self):
        return self.inv_freq
