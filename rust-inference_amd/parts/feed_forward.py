"""Feed-forward parts."""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, MATRIX, TensorSpec
from .base import FeedForward
from .registry import register_part


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))``, no bias, ``silu(z) = z / (1 + exp(-z))``
    (the reference: src/models/qwen3.rs:112-117; src/ops/elementwise.rs:9-12).  Gate and
    up are one product with the row-concatenated weight ``[gate; up]``."""

    links_norms = True

    def __init__(self, hidden: int, inter: int, prefix: str):
        self.hidden, self.inter, self.prefix = hidden, inter, prefix

    def tensors(self):
        p = self.prefix
        return {
            p + "gate_proj.weight": TensorSpec((self.inter, self.hidden), MATRIX),
            p + "up_proj.weight": TensorSpec((self.inter, self.hidden), MATRIX),
            p + "down_proj.weight": TensorSpec((self.hidden, self.inter), MATRIX),
        }

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        gate_up = rt.place_matrix(torch.cat([weights[p + "gate_proj.weight"], weights[p + "up_proj.weight"]], 0))
        self.w_gate_up = rt.pack(gate_up, swiglu=True)
        self.w_down = rt.pack(rt.place_matrix(weights[p + "down_proj.weight"]), parts_ok=True)

    def bind_plain(self, weights):
        p = self.prefix
        self.plain_w = {n: weights[p + n + "_proj.weight"].to(torch.float32).numpy() for n in ("gate", "up", "down")}

    def plain(self, x, ctx):
        from ..kernels import plain
        import numpy as np
        y = np.concatenate([plain.linear(x, self.plain_w["gate"]), plain.linear(x, self.plain_w["up"])], axis=1)
        return plain.linear(plain.swiglu(y), self.plain_w["down"])

    def takes_tiled_at(self, m: int) -> bool:
        """Whether this part's first product reads ``m`` rows in the matrix cores' order."""
        return self.rt.takes_tiled(self.w_gate_up, m)

    def forward(self, x, ctx, link=None):
        rt = self.rt
        # the activation is in the epilogue of the decode-size kernels, which hand the down product its rows
        # in the order it loads fastest when that product is a packed one too
        with profiler.section(profiler.MLP):
            a = rt.linear_packed(x, self.w_gate_up, tiled_out=rt.takes_tiled(self.w_down, x.shape[0], True))
            # may come in parts: the stream's next norm adds them
            return rt.linear_packed(a, self.w_down, parts_ok=True, link=link)


@register_part("feed_forward", "dense")
class DenseFF(FeedForward):
    """``down(act(up(x)))``, no gate and no bias; ``activation`` is one of ``ops.ACTIVATIONS`` (``"relu2"``:
    ``max(z, 0)^2``; ``"gelu_tanh"``: the tanh form of GELU).  ``names`` gives the checkpoint names of ``up`` and
    ``down`` where they are not ``<prefix>up_proj.weight`` and ``<prefix>down_proj.weight``."""

    def __init__(self, hidden: int, inter: int, prefix: str, names: dict | None = None, activation: str = "relu2"):
        if activation not in ops.ACTIVATIONS:
            raise ConfigError(f"activation {activation!r} is not one of {', '.join(sorted(ops.ACTIVATIONS))}")
        self.hidden, self.inter, self.prefix, self.activation = hidden, inter, prefix, activation
        self.names = {"up": prefix + "up_proj.weight", "down": prefix + "down_proj.weight"}
        self.names.update(names or {})

    def tensors(self):
        return {self.names["up"]: TensorSpec((self.inter, self.hidden), MATRIX),
                self.names["down"]: TensorSpec((self.hidden, self.inter), MATRIX)}

    def bind(self, weights, rt):
        self.rt = rt
        # like a gate|up pair, always with a packed copy: steps of 2 to 16 rows stream it three times as fast as the
        # library's product does a matrix of this size
        self.w_up = rt.pack(rt.place_matrix(weights[self.names["up"]]), always=True)
        self.w_down = rt.pack(rt.place_matrix(weights[self.names["down"]]), parts_ok=True)

    def forward(self, x, ctx):
        rt = self.rt
        with profiler.section(profiler.MLP):
            a = ops.ACTIVATIONS[self.activation](ops.as_rows(rt.linear_packed(x, self.w_up)))
            # float32 into the residual (or in parts that the stream's next read adds): the sum is never rounded to 16 bits
            return rt.linear_packed(a, self.w_down, out_dtype=torch.float32, parts_ok=True)


@register_part("feed_forward", "glu_clamped")
class ClampedGatedFF(FeedForward):
    """``down(g sigmoid(1.702 g) (u + 1))`` with ``g = min(gate(x), limit)`` and ``u = clamp(up(x), -limit, limit)``; with
    ``biases`` every product has one (``<name>.b``).  Gate and up are one product with the row-concatenated weight; their
    biases, the clamps and the activation are one kernel; the bias of the last product is offered to the residual
    stream (``out_bias``), which adds it where it adds the product.  ``names`` gives the checkpoint names of ``gate``,
    ``up`` and ``down`` where they are not ``<prefix>gate`` and so on."""

    def __init__(self, hidden: int, inter: int, limit: float, prefix: str, biases: bool = True, names: dict | None = None):
        if not limit > 0:
            raise ConfigError(f"the limit {limit} of a clamped feed-forward must be positive")
        self.hidden, self.inter, self.limit, self.prefix, self.biases = hidden, inter, float(limit), prefix, bool(biases)
        self.names = {"gate": prefix + "gate", "up": prefix + "up", "down": prefix + "down"}
        self.names.update(names or {})
        self.out_bias = None

    def tensors(self):
        n = self.names
        t = {n["gate"]: TensorSpec((self.inter, self.hidden), MATRIX), n["up"]: TensorSpec((self.inter, self.hidden), MATRIX),
             n["down"]: TensorSpec((self.hidden, self.inter), MATRIX)}
        if self.biases:
            t.update({n["gate"] + ".b": TensorSpec((self.inter,), BIAS), n["up"] + ".b": TensorSpec((self.inter,), BIAS),
                      n["down"] + ".b": TensorSpec((self.hidden,), BIAS)})
        return t

    def bind(self, weights, rt):
        self.rt = rt
        n = self.names
        self.w_gate_up = rt.pack(rt.place_matrix(torch.cat([weights[n["gate"]], weights[n["up"]]], 0)), always=True)
        self.w_down = rt.pack(rt.place_matrix(weights[n["down"]]), parts_ok=True)
        self.b_gate = rt.place_gain(weights[n["gate"] + ".b"]) if self.biases else None
        self.b_up = rt.place_gain(weights[n["up"] + ".b"]) if self.biases else None
        self.out_bias = rt.place_gain(weights[n["down"] + ".b"]) if self.biases else None

    def forward(self, x, ctx):
        rt = self.rt
        with profiler.section(profiler.MLP):
            gu = ops.as_rows(rt.linear_packed(x, self.w_gate_up))
            a = ops.glu_clamped_bias(gu, self.b_gate, self.b_up, self.limit)
            # float32 into the residual (or in parts that the stream's next read adds); the last bias rides as out_bias
            return rt.linear_packed(a, self.w_down, out_dtype=torch.float32, parts_ok=True)


@register_part("feed_forward", "relu2")
class ReluSquaredFF(DenseFF):
    """``down(relu(up(x))^2)``: the dense feed-forward with the squared ReLU."""

    def __init__(self, hidden: int, inter: int, prefix: str, names: dict | None = None):
        super().__init__(hidden, inter, prefix, names, "relu2")
