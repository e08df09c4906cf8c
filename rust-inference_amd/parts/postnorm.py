"""The arrangement whose norm sits behind the residual sum."""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from .parallel import NormAfterBlock
from .registry import register_part


@register_part("arrangement", "norm_after_sum")
class PostNormBlock(NormAfterBlock):
    """``x <- norm1(alpha x + mixer(x))``, then ``x <- norm2(alpha x + ff(x))``: the sublayers read the residual itself, and
    the residual is a norm's output (a post-norm layer with a constant on the skip path).  Parts: ``mixer``,
    ``mixer_norm`` and, for a layer with a feed-forward, ``feed_forward`` and ``feed_forward_norm``; the norms are of a kind
    with a gain and optionally a bias (``layernorm``, ``rmsnorm``); ``alpha`` is a parameter of the part ``"skip"``.

    The residual is float32; one kernel (``ops.scaled_sum_norm``) scales it, adds the sublayer's output (the parts of a
    split product in order, and the bias of the product that made it, which a sublayer offers as ``out_bias``), norms the
    sum and writes it back together with its copy in the activations' format, which the next sublayer's products read.
    A mixer that sets ``wants_residual`` also gets the float32 residual itself (``residual=``): what it keeps of its input
    from token to token is then not rounded."""

    def __init__(self, layer_spec):
        super().__init__(layer_spec)
        if self.scales is not None:
            raise ConfigError("a layer whose norm sits behind the sum has no layer scale")
        self.alpha = float(layer_spec.parts["skip"].params.get("alpha", 1.0)) if "skip" in layer_spec.parts else 1.0

    def parts(self):
        out = [self.mixer, self.mixer_norm]
        if self.feed_forward is not None:
            out += [self.feed_forward, self.feed_forward_norm]
        return tuple(out)

    def _close(self, stream, y, norm, sublayer, act_dtype):
        if isinstance(y, tuple):
            raise ConfigError("a sublayer in front of a norm behind the sum hands back its result, not a link to a norm")
        with profiler.section(profiler.NORM):
            y = ops.as_rows(y) if not isinstance(y, torch.Tensor) else y
            stream.as_act = ops.scaled_sum_norm(stream.sum, y, getattr(sublayer, "out_bias", None), self.alpha, norm.gain,
                                                getattr(norm, "bias", None), norm.eps, norm.kind,
                                                None if act_dtype == torch.float32 else act_dtype)

    def forward(self, stream, ctx, store, page_table, act_dtype) -> None:
        h = self._input(stream, act_dtype)
        if getattr(self.mixer, "wants_residual", False):
            y = self.mixer.forward(h, ctx, store, page_table, residual=stream.sum)
        else:
            y = self.mixer.forward(h, ctx, store, page_table)
        self._close(stream, y, self.mixer_norm, self.mixer, act_dtype)
        if self.feed_forward is not None:
            h = self._input(stream, act_dtype)
            self._close(stream, self.feed_forward.forward(h, ctx), self.feed_forward_norm, self.feed_forward, act_dtype)
