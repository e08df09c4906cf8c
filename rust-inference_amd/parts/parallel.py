"""Mixers side by side, and the arrangement whose norms sit on the sublayers' outputs."""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, TensorSpec
from .base import Mixer
from .registry import build_part, register_part


@register_part("mixer", "parallel")
class ParallelMixers(Mixer):
    """Several mixers that read the same input; the result is the sum of theirs, each times a constant:
    ``y = sum_i scale_i * mixer_i(h)``.  ``mixers``: a tuple of ``PartSpec`` (mixer kinds), ``scales``: as many numbers.

    Each member keeps what it keeps per sequence: ``cache_need()`` is the tuple of the members' needs, and the layer's
    run names as many cache entries.  Members that can be taken apart into an input product, a core and an output
    product (``in_matrix``, ``core``, ``out_matrix``: the attention of the third family, the linear attention with a
    fixed decay) share both products: one product with all members' input rows, the members' cores write their heads,
    times their constant, side by side into one row, and one product with the output matrices side by side along K
    adds the members up in its float32 sum.  Members that make their own input products but can write their finished heads
    into a row of another's (``run_into`` and ``out_matrix``: an attention whose heads talk, time mixing, whose five
    projections each read a mix of their own) share the output product alone.  Other members run whole, and their float32
    results are added.

    A member that keeps several things per sequence (a tuple of needs) gets its stores as a tuple; the layer's run names
    the members' entries one after the other.  A member that sets ``wants_residual`` also gets the float32 residual the
    layer hands over (``residual=``)."""

    wants_residual = True

    def __init__(self, mixers: tuple, scales: tuple):
        if len(mixers) < 1 or len(mixers) != len(scales):
            raise ConfigError(f"{len(mixers)} mixers side by side with {len(scales)} constants")
        self.members = [build_part("mixer", m) for m in mixers]
        self.scales = tuple(float(s) for s in scales)
        self.fused = all(hasattr(m, "core") and hasattr(m, "in_matrix") and hasattr(m, "out_matrix") and
                         (getattr(m, "paired", True)) for m in self.members)
        # members that write their heads into one row for one output product, each after input products of its own
        self.shares_out = not self.fused and all(hasattr(m, "run_into") and hasattr(m, "out_matrix") for m in self.members)

    def tensors(self):
        t = {}
        for m in self.members:
            t.update(m.tensors())
        return t

    def bind(self, weights, rt):
        self.rt = rt
        if self.shares_out:
            for m in self.members:
                m.bind(weights, rt, alone=False)
            self.w_out = rt.pack(rt.place_matrix(torch.cat([m.out_matrix(weights) for m in self.members], 1)), parts_ok=True)
            self.out_at, b = [], 0
            for m in self.members:
                self.out_at.append(b)
                b += m.out_width
            self.out_width = b
            return
        if not self.fused:
            for m in self.members:
                m.bind(weights, rt)
            return
        for m in self.members:
            m.bind(weights, rt, alone=False)
        self.w_in = rt.pack(rt.place_matrix(torch.cat([m.in_matrix(weights) for m in self.members], 0)), always=True)
        self.w_out = rt.pack(rt.place_matrix(torch.cat([m.out_matrix(weights) for m in self.members], 1)), parts_ok=True)
        self.in_at, self.out_at, a, b = [], [], 0, 0
        for m in self.members:
            self.in_at.append(a)
            self.out_at.append(b)
            a, b = a + m.in_width, b + m.out_width
        self.out_width = b

    def cache_need(self):
        needs = []
        for m in self.members:
            need = m.cache_need()
            needs += list(need) if isinstance(need, (tuple, list)) else [need]
        return tuple(needs)

    def _per_member(self, stores, page_tables):
        """The stores and page tables of a run, dealt out to the members: one each, or a tuple for a member with several needs."""
        out, at = [], 0
        for m in self.members:
            need = m.cache_need()
            if isinstance(need, (tuple, list)):
                out.append((tuple(stores[at:at + len(need)]), tuple(page_tables[at:at + len(need)])))
                at += len(need)
            else:
                out.append((stores[at], page_tables[at]))
                at += 1
        return out

    def forward(self, x, ctx, stores, page_tables, residual=None):
        rt = self.rt
        if not isinstance(stores, tuple):
            stores, page_tables = (stores,), (page_tables,)
        dealt = self._per_member(stores, page_tables)
        extra = lambda m: {"residual": residual} if getattr(m, "wants_residual", False) else {}
        if self.shares_out:
            rows = x.shape[0]
            heads = torch.empty((rows, self.out_width), dtype=rt.dtype, device=rt.device)
            for m, scale, (store, table), b in zip(self.members, self.scales, dealt, self.out_at):
                m.run_into(x, ctx, store, table, heads, b, scale, **extra(m))
            with profiler.section(profiler.OUT_PROJECTION):
                return rt.linear_packed(heads, self.w_out, out_dtype=torch.float32, parts_ok=True)
        if not self.fused:
            total = None
            for m, scale, (store, table) in zip(self.members, self.scales, dealt):
                y = m.forward(x, ctx, store, table, **extra(m))
                if isinstance(y, tuple):
                    raise ConfigError("a mixer side by side with others hands back its result, not a link to a norm")
                if y.dim() == 3:
                    y = ops.sum_parts(y, torch.float32)
                y = y.to(torch.float32) * scale
                total = y if total is None else total + y
            return total
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_in))
        heads = torch.empty((proj.shape[0], self.out_width), dtype=proj.dtype, device=proj.device)
        for m, scale, (store, table), a, b in zip(self.members, self.scales, dealt, self.in_at, self.out_at):
            m.core(proj, a, ctx, store, table, heads, b, scale)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(heads, self.w_out, out_dtype=torch.float32, parts_ok=True)


@register_part("arrangement", "norm_after")
class NormAfterBlock:
    """``x <- x + s1 * norm1(mixer(x))``, then ``x <- x + s2 * norm2(ff(x))``: the sublayers read the residual itself
    and the norm sits on each sublayer's output; ``s1`` and ``s2`` are learned vectors (a layer scale), read from the
    tensors ``scale_names`` names, or absent.  Parts: ``mixer``, ``mixer_norm`` and, for a layer with a feed-forward,
    ``feed_forward`` and ``feed_forward_norm``; the norms are of a kind with a gain and optionally a bias (``layernorm``,
    ``rmsnorm``).

    The residual is float32; one kernel (``ops.branch_norm_add``) norms a sublayer's output, scales it, adds it to the
    residual and writes the copy of the new residual in the activations' format that the next sublayer's products
    read.  That copy rides on the stream (``stream.as_act``) from layer to layer."""

    def __init__(self, layer_spec):
        self.mixer = build_part("mixer", layer_spec.mixer)
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm)
        self.feed_forward = self.feed_forward_norm = None
        if "feed_forward" in layer_spec.parts:
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward)
            self.feed_forward_norm = build_part("norm", layer_spec.feed_forward_norm)
        self.scales = LayerScales(layer_spec.parts["scales"].params) if "scales" in layer_spec.parts else None

    def parts(self):
        out = [self.mixer, self.mixer_norm]
        if self.feed_forward is not None:
            out += [self.feed_forward, self.feed_forward_norm]
        if self.scales is not None:
            out.append(self.scales)
        return tuple(out)

    def cache_need(self):
        return self.mixer.cache_need()

    def _input(self, stream, act_dtype):
        """The residual in the format the products read."""
        if stream.pending is not None or stream.later is not None:      # another arrangement's branch: the copy is stale
            stream.flush()
            stream.as_act = None
        if act_dtype == torch.float32:
            return stream.sum
        act = getattr(stream, "as_act", None)
        if act is None:                                   # the first layer: the residual as it is, in the products' format
            rows, dim = stream.sum.shape
            act = ops.streams_read_norm(stream.sum.view(rows, 1, dim), None, None, None, None, None, None, 0.0,
                                        ops.NORM_NONE, act_dtype, None)
        return act

    def _close(self, stream, y, norm, scale, act_dtype):
        if isinstance(y, tuple):
            raise ConfigError("a sublayer whose norm sits on its output hands back its result, not a link to a norm")
        with profiler.section(profiler.NORM):
            stream.as_act = ops.branch_norm_add(stream.sum, ops.as_rows(y) if not isinstance(y, torch.Tensor) else y,
                                                norm.gain, getattr(norm, "bias", None), norm.eps, norm.kind, scale,
                                                None if act_dtype == torch.float32 else act_dtype)

    def forward(self, stream, ctx, store, page_table, act_dtype) -> None:
        h = self._input(stream, act_dtype)
        s = self.scales
        self._close(stream, self.mixer.forward(h, ctx, store, page_table), self.mixer_norm, s.first if s else None, act_dtype)
        if self.feed_forward is not None:
            h = self._input(stream, act_dtype)
            self._close(stream, self.feed_forward.forward(h, ctx), self.feed_forward_norm, s.second if s else None, act_dtype)


class LayerScales:
    """The two learned vectors of a layer scale, ``names = (first, second)`` (the second may be None)."""

    def __init__(self, params: dict):
        self.dim, self.names = params["dim"], tuple(params["names"])

    def tensors(self):
        return {n: TensorSpec((self.dim,), GAIN) for n in self.names if n}

    def bind(self, weights, rt):
        self.rt = rt
        self.first = rt.place_gain(weights[self.names[0]]) if self.names[0] else None
        self.second = rt.place_gain(weights[self.names[1]]) if len(self.names) > 1 and self.names[1] else None
