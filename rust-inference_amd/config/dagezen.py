"""Configuration of the Dagezen decoder, from its config.json.

A Dagezen model is a list of layers whose norm sits behind the residual sum: ``x <- norm(alpha x + sublayer(x))``.  A
layer's mixer is one of three: a state-space mixer with a scalar decay per head (``"mamba2"``), attention over a cached
latent (``"latent_attention"``), or two mixers side by side (``"parallel"``): a windowed attention whose values are its
keys and whose heads talk after the softmax, and time mixing with a decay per channel.  Its feed-forward is dense with
a clamped gate, or a mixture of experts without gates.  The logits are capped.  config.json names the design in
``"architecture"`` and gives every size and constant:

    vocab, width, norm: {eps}, postln_alpha, logit_softcap,
    layers: [{type: "mamba2", mixer: {heads, vdim, state, groups, conv, norm_groups}, mlp}
             {type: "latent_attention", mixer: {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {dims, base}}, mlp}
             {type: "parallel", mixer: {left: {heads, kv_heads, dim, vdim, scale, mask: {size}}, right: {heads, dim[, rank]},
                                        left_scale, right_scale}, mlp}, ...]
    mlp: {kind: "dense", ff, limit} or {kind: "moe", expert: {ff}, router: {experts, top}} or null

``max_positions`` is no key of the design (positions enter through angles and distances alone); where it is given it
is the default length of a cache that is given none.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar, Optional

from ..errors import ConfigError, UnsupportedError
from .base import ModelConfig, f32, whole

DEFAULT_MAX_POSITIONS = 1 << 20


def _section(raw, key: str, where: str) -> dict:
    v = raw.get(key) if isinstance(raw, dict) else None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: {key!r} must be an object, got {v!r}")
    return v


def _need(m: dict, keys: tuple, where: str) -> None:
    missing = [k for k in keys if k not in m]
    if missing:
        raise ConfigError(f"{where} lacks {', '.join(missing)}")


@dataclass(frozen=True)
class StateSpaceSizes:
    heads: int
    vdim: int                         # channels of a head
    state: int                        # rows of a head's state
    groups: int                       # groups of heads that share B and C
    conv: int                         # taps of the short convolution
    norm_groups: int                  # equal parts of the output that are normed each on its own

    @classmethod
    def read(cls, m: dict, where: str) -> "StateSpaceSizes":
        _need(m, ("heads", "vdim", "state"), where)
        heads = whole(m["heads"], where + ".heads", 1)
        groups = whole(m.get("groups", 1), where + ".groups", 1)
        vdim = whole(m["vdim"], where + ".vdim", 1)
        parts = whole(m.get("norm_groups", 1), where + ".norm_groups", 1)
        if heads % groups:
            raise ConfigError(f"{where}: {heads} heads not divisible by {groups} groups")
        if (heads * vdim) % parts:
            raise ConfigError(f"{where}: {heads * vdim} channels not divisible into {parts} normed parts")
        return cls(heads, vdim, whole(m["state"], where + ".state", 1), groups, whole(m.get("conv", 1), where + ".conv", 1), parts)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int                          # unrotated elements of a query or key head
    rot_dim: int                      # rotated elements, shared by the heads on the key side
    vdim: int
    kv_rank: int                      # size of the cached latent
    scale: float
    rot_dims: int                     # how many of the rotated elements turn (the design: all of them)
    rot_base: float

    @classmethod
    def read(cls, m: dict, where: str) -> "LatentAttentionSizes":
        _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"), where)
        rot_dim = whole(m["rot_dim"], where + ".rot_dim", 0)
        rot_dims, base = rot_dim, 10000.0
        if m.get("rot") is not None:
            rot = _section(m, "rot", where)
            rot_dims = whole(rot.get("dims", rot_dim), where + ".rot.dims", 0)
            base = f32(rot.get("base", base), where + ".rot.base")
        if rot_dims % 2 or rot_dims > rot_dim:
            raise ConfigError(f"{where}.rot.dims {rot_dims} must be even and at most rot_dim {rot_dim}")
        if rot_dims and not base > 0:
            raise ConfigError(f"{where}.rot.base {base} must be positive")
        return cls(whole(m["heads"], where + ".heads", 1), whole(m["dim"], where + ".dim", 0), rot_dim,
                   whole(m["vdim"], where + ".vdim", 1), whole(m["kv_rank"], where + ".kv_rank", 1),
                   f32(m["scale"], where + ".scale"), rot_dims, base)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": {"dims": self.rot_dims, "base": self.rot_base}}


@dataclass(frozen=True)
class TalkingAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int                         # the values are the keys: it equals dim
    scale: float
    window: Optional[int]             # a query at i sees j with 0 <= i - j < window; None: all

    @classmethod
    def read(cls, m: dict, where: str) -> "TalkingAttentionSizes":
        _need(m, ("heads", "dim", "scale"), where)
        heads = whole(m["heads"], where + ".heads", 1)
        kv = whole(m.get("kv_heads", heads), where + ".kv_heads", 1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads not divisible by {kv} kv heads")
        dim = whole(m["dim"], where + ".dim", 1)
        vdim = whole(m.get("vdim", dim), where + ".vdim", 1)
        if vdim != dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim {vdim} must equal dim {dim}")
        window = None
        if m.get("mask") is not None and _section(m, "mask", where).get("size") is not None:
            window = whole(m["mask"]["size"], where + ".mask.size", 1)
        return cls(heads, kv, dim, vdim, f32(m["scale"], where + ".scale"), window)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class TimeMixSizes:
    heads: int
    dim: int
    rank: Optional[int] = None        # the narrow middle of the decay's two products; None: the checkpoint gives it

    @classmethod
    def read(cls, m: dict, where: str) -> "TimeMixSizes":
        _need(m, ("heads", "dim"), where)
        rank = whole(m["rank"], where + ".rank", 1) if m.get("rank") is not None else None
        return cls(whole(m["heads"], where + ".heads", 1), whole(m["dim"], where + ".dim", 1), rank)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class SideBySideSizes:
    left: TalkingAttentionSizes
    right: TimeMixSizes
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, m: dict, where: str) -> "SideBySideSizes":
        return cls(TalkingAttentionSizes.read(_section(m, "left", where), where + ".left"),
                   TimeMixSizes.read(_section(m, "right", where), where + ".right"),
                   f32(m.get("left_scale", 1.0), where + ".left_scale"), f32(m.get("right_scale", 1.0), where + ".right_scale"))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class ClampedDenseSizes:
    ff: int
    limit: float

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class PlainExpertsSizes:
    experts: int
    top: int
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


def _read_mlp(entry: dict, where: str):
    if entry.get("mlp") is None:
        return None
    mlp = _section(entry, "mlp", where)
    kind = mlp.get("kind")
    if kind == "dense":
        limit = f32(mlp.get("limit"), where + ".mlp.limit")
        if not limit > 0:
            raise ConfigError(f"{where}.mlp.limit {limit} must be positive")
        return ClampedDenseSizes(whole(mlp.get("ff"), where + ".mlp.ff", 1), limit)
    if kind == "moe":
        expert, router = _section(mlp, "expert", where + ".mlp"), _section(mlp, "router", where + ".mlp")
        experts = whole(router.get("experts"), where + ".mlp.router.experts", 1)
        top = whole(router.get("top"), where + ".mlp.router.top", 1)
        if top > experts:
            raise ConfigError(f"{where}.mlp.router: the {top} best of {experts} experts")
        return PlainExpertsSizes(experts, top, whole(expert.get("ff"), where + ".mlp.expert.ff", 1))
    raise UnsupportedError(f"{where}: feed-forward kind {kind!r} is neither 'dense' nor 'moe'")


MIXER_SIZES = {"mamba2": StateSpaceSizes, "latent_attention": LatentAttentionSizes, "parallel": SideBySideSizes}


@dataclass(frozen=True)
class DagezenLayer:
    type: str                                     # a key of MIXER_SIZES
    mixer: object
    mlp: object = None                            # ClampedDenseSizes, PlainExpertsSizes or None: no feed-forward

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class DagezenConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: tuple = ()
    norm_eps: float = 1e-5
    postln_alpha: float = 1.0
    logit_softcap: Optional[float] = None
    max_positions: int = DEFAULT_MAX_POSITIONS

    ARCHITECTURE: ClassVar[str] = "Dagezen"
    MODEL_TYPE: ClassVar[str] = "dagezen"
    REQUIRED: ClassVar[tuple[str, ...]] = ("vocab", "width", "layers", "norm")

    @classmethod
    def from_dict(cls, raw: dict) -> "DagezenConfig":
        cls.require(raw)
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config key 'layers' must be a list of at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else entry
            if kind not in MIXER_SIZES:
                raise UnsupportedError(f"{where}: mixer type {kind!r} is none of {', '.join(sorted(MIXER_SIZES))}")
            layers.append(DagezenLayer(kind, MIXER_SIZES[kind].read(_section(entry, "mixer", where), where + ".mixer"),
                                       _read_mlp(entry, where)))
        cap = raw.get("logit_softcap")
        cfg = cls(vocab=whole(raw["vocab"], "vocab", 1), width=whole(raw["width"], "width", 1), layers=tuple(layers),
                  norm_eps=f32(_section(raw, "norm", "config.json").get("eps"), "norm.eps"),
                  postln_alpha=f32(raw.get("postln_alpha", 1.0), "postln_alpha"),
                  logit_softcap=f32(cap, "logit_softcap") if cap else None,
                  max_positions=whole(raw.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions", 1))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"norm.eps {self.norm_eps} must not be negative")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"logit_softcap {self.logit_softcap} must be positive")

    def to_dict(self) -> dict:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "postln_alpha": self.postln_alpha, "layers": [layer.to_dict() for layer in self.layers]}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out
