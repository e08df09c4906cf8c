"""A mixture of experts as a feed-forward part."""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, MATRIX, TensorSpec
from .base import FeedForward
from .registry import register_part


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """``experts`` small feed-forward layers of which every token uses ``top``.

    Router: logits ``z = W_router h`` in float32, scores ``s = sigmoid(z)``; the ``top`` experts with the largest
    ``s + correction`` are chosen, and their weights are their scores ``s`` (without the correction) divided by the
    sum of the chosen scores (+ 1e-20).  Expert: ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, -limit, limit)``,
    output ``W_down (g sigmoid(1.702 g) (u + 1))``; no biases.  The part's output is the weighted sum of the chosen
    experts' outputs.

    The experts' matrices lie as two: every expert's gate and up rows side by side (``[experts, 2, ff]`` rows), and
    every expert's down matrix side by side along K.  A step of a few tokens reads only the rows of the experts
    chosen; a prompt sorts its tokens by expert and runs two products an expert; in between (and in float32) the two
    matrices are two products over all tokens, between which the activation kernel writes zeros for the experts a
    token did not choose and the router's weight times the activation for those it did, so that the second product's
    sum over K is the weighted sum.  The three differ by rounding alone.

    Tensors: ``<prefix>router [experts, hidden]``, ``<prefix>correction [experts]``, ``<prefix>e<i>.gate`` / ``.up``
    ``[ff, hidden]``, ``<prefix>e<i>.down [hidden, ff]``.

    Other routers and experts, by parameter.  ``scores="softmax"``: ``s`` is the softmax over all of the router's
    outputs.  ``normalize=False``: the weights are the chosen ``s`` themselves.  ``groups=(count, keep)``: the outputs
    form ``count`` equal groups of neighbours, a group's score is its largest ``s + correction``, and only outputs of the
    ``keep`` best groups can be chosen.  ``identity=n``: the router has ``n`` more outputs after the experts', which
    stand for experts that hand the token's own row on (times the weight) and have no tensors; they are scored,
    grouped and chosen like the others.  ``limit=None``: an expert is ``W_down (silu(W_gate h) (W_up h))``.
    ``gated=False, activation=...``: an expert is ``W_down act(W_up h)`` (``<prefix>e<i>.up`` and ``.down`` alone), ``act`` one of
    ``ops.PLAIN_ACTIVATIONS``.  ``router_bias=True``: the logits are ``W_router h + b`` (``<prefix>router.b``) and there is no
    correction; with ``scores="softmax"`` and ``normalize=True`` the weights are then the softmax over the chosen logits alone.
    ``shared=ff``: one more expert of that width and form, ``<prefix>shared.gate`` / ``.up`` / ``.down``, runs for
    every token and is added times ``sigmoid(W_sg h)``, one number a token (``<prefix>shared.sg [1, hidden]``; its row
    rides as the last row of the router's matrix).
    """

    def __init__(self, hidden: int, inter: int, experts: int, top: int, limit: float | None, prefix: str,
                 scores: str = "sigmoid", normalize: bool = True, groups: tuple | None = None, identity: int = 0,
                 shared: int | None = None, gated: bool = True, activation: str | None = None, router_bias: bool = False):
        self.outs = experts + int(identity)
        self.gated, self.activation, self.router_bias = bool(gated), activation, bool(router_bias)
        if not self.gated:
            if activation not in ops.PLAIN_ACTIVATIONS:
                raise ConfigError(f"experts without a gate name one of {', '.join(sorted(ops.PLAIN_ACTIVATIONS))}, not {activation!r}")
            if identity or shared is not None or limit is not None:
                raise ConfigError("experts without a gate take no limit, no identity experts and no shared expert")
        if not 1 <= top <= self.outs <= ops.EXPERTS_MAX or experts < 1:
            raise ConfigError(f"the {top} best of {experts} experts and {identity} identity experts: the router takes up to "
                              f"{ops.EXPERTS_MAX} outputs")
        if limit is not None and not limit > 0:
            raise ConfigError(f"the experts' limit {limit} must be positive")
        if scores not in ("sigmoid", "softmax"):
            raise ConfigError(f"router scores {scores!r} are neither 'sigmoid' nor 'softmax'")
        self.hidden, self.inter, self.experts, self.top, self.prefix = hidden, inter, experts, top, prefix
        self.limit = float(limit) if limit is not None else 0.0          # 0: the plain gated form
        self.scores, self.normalize, self.identity, self.shared = scores, bool(normalize), int(identity), shared
        self.groups, self.keep = (int(groups[0]), int(groups[1])) if groups else (1, 1)
        if self.outs % self.groups or not 1 <= self.keep <= self.groups or top > self.keep * (self.outs // self.groups):
            raise ConfigError(f"{self.outs} router outputs in {self.groups} groups of which {self.keep} stay, for the {top} best")
        # the router of the first designs: one kernel call and no extras
        self.simple = (scores == "sigmoid" and self.normalize and self.groups == 1 and not self.identity and shared is None)

    def tensors(self):
        p, t = self.prefix, {}
        t[p + "router"] = TensorSpec((self.outs, self.hidden), MATRIX)
        if self.router_bias:
            t[p + "router.b"] = TensorSpec((self.outs,), BIAS)
        else:
            t[p + "correction"] = TensorSpec((self.outs,), BIAS)
        if self.shared is not None:
            t[p + "shared.gate"] = TensorSpec((self.shared, self.hidden), MATRIX)
            t[p + "shared.up"] = TensorSpec((self.shared, self.hidden), MATRIX)
            t[p + "shared.down"] = TensorSpec((self.hidden, self.shared), MATRIX)
            t[p + "shared.sg"] = TensorSpec((1, self.hidden), MATRIX)
        for e in range(self.experts):
            if self.gated:
                t[f"{p}e{e}.gate"] = TensorSpec((self.inter, self.hidden), MATRIX)
            t[f"{p}e{e}.up"] = TensorSpec((self.inter, self.hidden), MATRIX)
            t[f"{p}e{e}.down"] = TensorSpec((self.hidden, self.inter), MATRIX)
        return t

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        router = weights[p + "router"]
        if self.shared is not None:                       # the shared expert's gate: one more row of logits
            router = torch.cat([router, weights[p + "shared.sg"].to(router.dtype)], 0)
            self.w_shared_in = rt.pack(rt.place_matrix(torch.cat([weights[p + "shared.gate"], weights[p + "shared.up"]], 0)),
                                       swiglu=True)
            self.w_shared_down = rt.pack(rt.place_matrix(weights[p + "shared.down"]), parts_ok=True)
        self.w_router = rt.pack(rt.place_matrix(router))
        if self.router_bias:
            # a bias of the router's product: it moves the logits themselves, so choice and weights both see it
            self.z_bias = rt.place_gain(weights[p + "router.b"])
            self.correction = torch.zeros_like(self.z_bias)
        else:
            self.z_bias, self.correction = None, rt.place_gain(weights[p + "correction"])
        rows = []
        for e in range(self.experts):
            rows += [weights[f"{p}e{e}.gate"], weights[f"{p}e{e}.up"]] if self.gated else [weights[f"{p}e{e}.up"]]
        self.w_gate_up = rt.pack(rt.place_matrix(torch.cat(rows, 0)), always=True)
        down = torch.cat([weights[f"{p}e{e}.down"] for e in range(self.experts)], 1)
        self.w_down = rt.pack(rt.place_matrix(down), parts_ok=True)

    # A step with fewer assignments (tokens x top) than experts reads only the rows of the experts its tokens chose
    # (one wavefront an output row: every assignment streams its expert's matrices once, so with as many assignments
    # as experts it would read what all experts hold); from SORTED_MIN_TOKENS tokens on a prompt's assignments are
    # sorted by expert and every expert is two library products over its own rows; between them, and in float32, all
    # experts are computed for all tokens as two products, with zeros where a token did not choose.
    SORTED_MIN_TOKENS = 256

    def forward(self, x, ctx):
        rt = self.rt
        with profiler.section(profiler.MLP):
            z = ops.as_rows(rt.linear_packed(x, self.w_router, out_dtype=torch.float32))
            if self.z_bias is not None:
                z = ops.add_bias(z, self.z_bias)
            extra = None
            if self.simple:
                ids, weights, dense = ops.experts_route(z, self.correction, self.top)
            else:
                ids, weights, dense, extra = ops.experts_route_general(
                    z, self.correction, self.outs, self.experts, self.top,
                    ops.ROUTE_SOFTMAX if self.scores == "softmax" else ops.ROUTE_SIGMOID, self.normalize, self.groups, self.keep)
            tokens = z.shape[0]
            routed = (rt.dtype == torch.bfloat16 and not rt.invariant and self.top < self.experts
                      and self.hidden % 8 == 0 and self.inter % 8 == 0)
            few = routed and self.gated          # the kernel that reads the chosen experts' rows alone knows gated experts
            own = self.identity > 0                   # whether the identity experts' share is still to be added
            if few and tokens * self.top < self.experts:
                y, own = ops.experts_few_tokens(rt.normed_now(x), self.w_gate_up.w, self.w_down.w, ids, weights, self.inter,
                                                self.limit), False
            elif (routed and tokens >= self.SORTED_MIN_TOKENS and not ctx.is_decode
                    and not torch.cuda.is_current_stream_capturing()):
                y, own = self.forward_sorted(rt.normed_now(x), ids, weights), False
            else:
                gu = ops.as_rows(rt.linear_packed(x, self.w_gate_up))
                a = (ops.experts_activate(gu, dense, self.inter, self.limit) if self.gated
                     else ops.experts_activate_plain(gu, dense, self.inter, self.activation))
                # float32 into the residual (or in parts that the stream's next read adds)
                y = rt.linear_packed(a, self.w_down, out_dtype=torch.float32, parts_ok=True)
            if not own and self.shared is None:
                return y
            shared = None
            if self.shared is not None:
                act = rt.linear_packed(x, self.w_shared_in)
                shared = rt.linear_packed(act, self.w_shared_down, out_dtype=torch.float32, parts_ok=True)
            return ops.experts_finish(y, rt.normed_now(x) if own else None, shared, extra)

    def forward_sorted(self, x, ids, weights):
        """A prompt: every expert's tokens as rows side by side, two library products an expert, the weighted sum in
        float32.  The host reads how many rows every expert has (one wait a layer), which a captured step could not."""
        ff = self.inter
        rows_each = 2 * ff if self.gated else ff
        dest, offsets = ops.experts_sort(ids, self.outs)
        rows = ops.experts_gather(x, dest, self.top)
        y = torch.empty_like(rows)
        starts = offsets.tolist()
        for e in range(self.experts):
            a, b = starts[e], starts[e + 1]
            if b > a:
                gu = torch.mm(rows[a:b], self.w_gate_up.w[e * rows_each:(e + 1) * rows_each].t())
                act = (ops.experts_activate(gu, None, ff, self.limit) if self.gated
                       else ops.experts_activate_plain(gu, None, ff, self.activation))
                torch.mm(act, self.w_down.w[:, e * ff:(e + 1) * ff].t(), out=y[a:b])
        if self.identity and starts[self.outs] > starts[self.experts]:
            y[starts[self.experts]:] = rows[starts[self.experts]:]        # identity experts: the token's own row
        return ops.experts_combine(y, dest, weights)
