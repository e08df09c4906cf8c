"""Zakelorn as a list of parts.

Embedding: the token's row times a constant.  Every layer reads the residual itself and norms its sublayers' outputs:
``x <- x + ls1 * norm1(mixer(x))``, ``x <- x + ls2 * norm2(ff(x))``, layer norms with gain and bias, ``ls`` learned vectors.
The mixer is two mixers side by side on the same input, added with a constant each: softmax attention (rotation of
neighbouring elements over the first part of a head, unit-normed q and k, a sliding window that keeps a sequence's
first tokens, a sink per head, a sigmoid output gate) and linear attention with a fixed decay per head (silu on q, k
and v, one RMS norm over all heads, a sigmoid output gate).  The feed-forward is dense with the tanh form of GELU or
a mixture of experts: softmax router, correction for the choice alone, groups, identity experts, weights not
renormalized, silu-gated experts, and an expert every token uses behind a sigmoid gate.  Final layer norm; the
output matrix is the embedding table.

Checkpoint names: ``embed``, ``l<i>.norm1`` / ``norm2`` (+ ``.b``), ``l<i>.ls1`` / ``ls2``, ``l<i>.mix.left.*`` /
``mix.right.*``, ``l<i>.mlp.*``, ``final.norm`` (+ ``.b``).
"""
from __future__ import annotations

from ..config import ZakelornConfig, register_architecture
from ..config.zakelorn import DenseSizes
from .spec import LayerSpec, ModelSpec, PartSpec, Run


def _norm(cfg: ZakelornConfig, name: str) -> PartSpec:
    return PartSpec("layernorm", {"dim": cfg.width, "eps": cfg.norm_eps, "name": name, "bias_name": name + ".b"})


def _mixer(cfg: ZakelornConfig, layer, p: str) -> PartSpec:
    m = layer.mixer
    a, r = m.left, m.right
    lp, rp = p + "left.", p + "right."
    left = PartSpec("attention", {
        "hidden": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "head_dim": a.dim, "v_dim": a.vdim, "prefix": lp,
        "qk_norm": "unit", "eps": cfg.norm_eps, "window": a.window, "keep_first": a.keep_first if a.window else 0,
        "scale": a.scale, "sinks": True, "gate": "sigmoid",
        "position": PartSpec("rotate_pairs", {"head_dim": a.dim, "dims": a.rot_dims, "base": a.rot_base}),
        "names": {"q": lp + "q", "k": lp + "k", "v": lp + "v", "o": lp + "o", "g": lp + "g", "sink": lp + "sink"},
    })
    right = PartSpec("decay_attention", {"hidden": cfg.width, "heads": r.heads, "dim": r.dim, "vdim": r.vdim,
                                         "decay": r.decay, "prefix": rp, "eps": cfg.norm_eps, "gate": "sigmoid"})
    return PartSpec("parallel", {"mixers": (left, right), "scales": (m.left_scale, m.right_scale)})


def _feed_forward(cfg: ZakelornConfig, mlp, p: str) -> PartSpec:
    if isinstance(mlp, DenseSizes):
        return PartSpec("dense", {"hidden": cfg.width, "inter": mlp.ff, "prefix": p, "activation": "gelu_tanh",
                                  "names": {"up": p + "up", "down": p + "down"}})
    return PartSpec("routed_experts", {"hidden": cfg.width, "inter": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                                       "limit": None, "prefix": p, "scores": "softmax", "normalize": False,
                                       "groups": (mlp.groups, mlp.keep), "identity": mlp.identity, "shared": mlp.shared_ff})


def zakelorn_spec(cfg: ZakelornConfig) -> ModelSpec:
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer": _mixer(cfg, layer, p + "mix."), "mixer_norm": _norm(cfg, p + "norm1")}
        second = None
        if layer.mlp is not None:
            parts["feed_forward"] = _feed_forward(cfg, layer.mlp, p + "mlp.")
            parts["feed_forward_norm"] = _norm(cfg, p + "norm2")
            second = p + "ls2"
        parts["scales"] = PartSpec("layer_scales", {"dim": cfg.width, "names": (p + "ls1", second)})
        layers.append(LayerSpec("norm_after", parts))
        schedule.append(Run(layer=i, cache=(2 * i, 2 * i + 1)))       # the attention's keys and values; the state
    return ModelSpec(
        architecture=cfg.ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("table", {"vocab": cfg.vocab, "dim": cfg.width, "name": "embed", "scale": cfg.embedding_scale}),
        layers=tuple(layers),
        schedule=tuple(schedule),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab": cfg.vocab, "dim": cfg.width, "name": "head", "tied": True}),
        max_positions=cfg.max_positions,
    )


register_architecture("Zakelorn", ZakelornConfig, zakelorn_spec, model_types=("zakelorn",))
