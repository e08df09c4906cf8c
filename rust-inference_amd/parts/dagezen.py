"""Dagezen as a list of parts.

Embedding: the token's row.  Every layer reads the residual itself and norms behind the sum:
``x <- norm1(alpha x + mixer(x))``, ``x <- norm2(alpha x + ff(x))``, layer norms with gain and bias.  The mixer is a
state-space mixer with a scalar decay per head, attention over a cached latent with a rotated part, a sink per head and
a gate per head, or two mixers side by side, added with a constant each: a windowed attention whose values are its keys
(q and k normed over the whole projection, a logarithmic distance bias, heads that talk after the softmax, a sigmoid
gate) and time mixing with a decay per channel.  The feed-forward is dense with a clamped gate and biases, or a mixture
of experts without gates (exact GELU) whose weights are the softmax over the chosen logits.  Final layer norm; the output
matrix is the embedding table, and the logits are capped.

Checkpoint names: ``embed``, ``l<i>.norm1`` / ``norm2`` (+ ``.b``), ``l<i>.mix.*`` (``mix.left.*`` / ``mix.right.*``),
``l<i>.mlp.*``, ``final.norm`` (+ ``.b``).
"""
from __future__ import annotations

from ..config import DagezenConfig, register_architecture
from ..config.dagezen import ClampedDenseSizes, LatentAttentionSizes, SideBySideSizes, StateSpaceSizes
from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, Run


def _norm(cfg: DagezenConfig, name: str) -> PartSpec:
    return PartSpec("layernorm", {"dim": cfg.width, "eps": cfg.norm_eps, "name": name, "bias_name": name + ".b"})


def _mixer(cfg: DagezenConfig, layer, p: str):
    """The mixer's part and how many things it keeps per sequence."""
    m = layer.mixer
    if isinstance(m, StateSpaceSizes):
        return PartSpec("state_space", {"hidden": cfg.width, "heads": m.heads, "vdim": m.vdim, "state": m.state,
                                        "groups": m.groups, "taps": m.conv, "norm_groups": m.norm_groups, "prefix": p,
                                        "eps": cfg.norm_eps}), 2
    if isinstance(m, LatentAttentionSizes):
        return PartSpec("latent_attention", {
            "hidden": cfg.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
            "scale": m.scale, "prefix": p, "eps": cfg.norm_eps, "sinks": True, "gate": True,
            "position": PartSpec("rotate_pairs", {"head_dim": m.rot_dim, "dims": m.rot_dims, "base": m.rot_base})}), 1
    if isinstance(m, SideBySideSizes):
        a, r = m.left, m.right
        left = PartSpec("talking_attention", {"hidden": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim,
                                              "scale": a.scale, "prefix": p + "left.", "eps": cfg.norm_eps, "window": a.window})
        right = PartSpec("time_mix", {"hidden": cfg.width, "heads": r.heads, "dim": r.dim, "prefix": p + "right.",
                                      "eps": cfg.norm_eps, "decay_rank": r.rank})
        return PartSpec("parallel", {"mixers": (left, right), "scales": (m.left_scale, m.right_scale)}), 3
    raise ConfigError(f"no mixer for {type(m).__name__}")


def _feed_forward(cfg: DagezenConfig, mlp, p: str) -> PartSpec:
    if isinstance(mlp, ClampedDenseSizes):
        return PartSpec("glu_clamped", {"hidden": cfg.width, "inter": mlp.ff, "limit": mlp.limit, "prefix": p, "biases": True})
    return PartSpec("routed_experts", {"hidden": cfg.width, "inter": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                                       "limit": None, "prefix": p, "scores": "softmax", "normalize": True, "gated": False,
                                       "activation": "gelu_erf", "router_bias": True})


def dagezen_spec(cfg: DagezenConfig) -> ModelSpec:
    layers, schedule, entry = [], [], 0
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mixer, kept = _mixer(cfg, layer, p + "mix.")
        parts = {"mixer": mixer, "mixer_norm": _norm(cfg, p + "norm1"), "skip": PartSpec("skip", {"alpha": cfg.postln_alpha})}
        if layer.mlp is not None:
            parts["feed_forward"] = _feed_forward(cfg, layer.mlp, p + "mlp.")
            parts["feed_forward_norm"] = _norm(cfg, p + "norm2")
        layers.append(LayerSpec("norm_after_sum", parts))
        schedule.append(Run(layer=i, cache=entry if kept == 1 else tuple(range(entry, entry + kept))))
        entry += kept
    return ModelSpec(
        architecture=cfg.ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("table", {"vocab": cfg.vocab, "dim": cfg.width, "name": "embed"}),
        layers=tuple(layers),
        schedule=tuple(schedule),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab": cfg.vocab, "dim": cfg.width, "name": "head", "tied": True,
                                 "softcap": cfg.logit_softcap}),
        max_positions=cfg.max_positions,
    )


register_architecture("Dagezen", DagezenConfig, dagezen_spec, model_types=("dagezen",))
