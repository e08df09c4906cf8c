"""Configuration of the Zakelorn decoder, from its config.json.

A Zakelorn model is a list of layers whose norms sit on the sublayers' outputs.  A layer's mixer is two mixers side by
side that read the same input: softmax attention with a rotation of neighbouring elements, unit-normed queries and
keys, a sliding window that keeps a sequence's first tokens, a sink per head and an output gate; and linear attention
with a fixed decay per head.  Its feed-forward is dense or a mixture of experts with a softmax router, groups,
identity experts and an expert that every token uses.  config.json names the design in ``"architecture"`` and gives
every size and constant:

    vocab, width, norm: {eps}, embedding: {scale},
    layers: [{type: "parallel",
              mixer: {left: {heads, kv_heads, dim, vdim, scale, rot: {dims, base}, mask: {size, keep_first}},
                      right: {heads, dim, vdim, decay: [one per head]}, left_scale, right_scale},
              mlp: {kind: "dense", ff}
                   or {kind: "moe", expert: {ff}, router: {experts, top, identity, groups: {count, keep}}, shared: {ff}}
                   or null}, ...]

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


@dataclass(frozen=True)
class WindowedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int                          # size of a query or key head
    vdim: int                         # size of a value head
    scale: float                      # factor on q . k
    rot_dims: int                     # the first rot_dims elements of a head turn, in neighbouring pairs
    rot_base: float
    window: Optional[int]             # a query at i sees j <= i with i - j < window; None: all
    keep_first: int                   # ... and every j < keep_first

    @classmethod
    def read(cls, m: dict, where: str) -> "WindowedAttentionSizes":
        for key in ("heads", "dim", "scale"):
            if key not in m:
                raise ConfigError(f"{where}: an attention mixer needs {key!r}")
        heads = whole(m["heads"], where + ".heads", 1)
        kv = whole(m.get("kv_heads", heads), where + ".kv_heads", 1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads not divisible by {kv} kv heads")
        dim = whole(m["dim"], where + ".dim", 1)
        rot_dims, rot_base = 0, 10000.0
        if m.get("rot") is not None:
            rot = _section(m, "rot", where)
            rot_dims = whole(rot.get("dims"), where + ".rot.dims", 0)
            rot_base = f32(rot.get("base"), where + ".rot.base")
            if rot_dims % 2 or rot_dims > dim:
                raise ConfigError(f"{where}.rot.dims {rot_dims} must be even and at most the head size {dim}")
            if rot_dims and not rot_base > 0:
                raise ConfigError(f"{where}.rot.base {rot_base} must be positive")
        window, keep = None, 0
        if m.get("mask") is not None:
            mask = _section(m, "mask", where)
            if mask.get("size") is not None:
                window = whole(mask["size"], where + ".mask.size", 1)
            keep = whole(mask.get("keep_first", 0), where + ".mask.keep_first", 0)
        return cls(heads, kv, dim, whole(m.get("vdim", dim), where + ".vdim", 1), f32(m["scale"], where + ".scale"),
                   rot_dims, rot_base, window, keep)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot_dims:
            out["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        if self.window is not None:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out


@dataclass(frozen=True)
class DecayAttentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: tuple                      # one per head

    @classmethod
    def read(cls, m: dict, where: str) -> "DecayAttentionSizes":
        for key in ("heads", "dim", "decay"):
            if key not in m:
                raise ConfigError(f"{where}: a linear-attention mixer needs {key!r}")
        heads = whole(m["heads"], where + ".heads", 1)
        dim = whole(m["dim"], where + ".dim", 1)
        decay = m["decay"] if isinstance(m["decay"], list) else [m["decay"]] * heads     # one number: the same for every head
        if len(decay) != heads:
            raise ConfigError(f"{where}.decay must list one decay for each of the {heads} heads")
        return cls(heads, dim, whole(m.get("vdim", dim), where + ".vdim", 1),
                   tuple(f32(d, where + ".decay") for d in decay))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class ParallelSizes:
    left: WindowedAttentionSizes
    right: DecayAttentionSizes
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, m: dict, where: str) -> "ParallelSizes":
        return cls(WindowedAttentionSizes.read(_section(m, "left", where), where + ".left"),
                   DecayAttentionSizes.read(_section(m, "right", where), where + ".right"),
                   f32(m.get("left_scale", 1.0), where + ".left_scale"), f32(m.get("right_scale", 1.0), where + ".right_scale"))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class GroupedExpertsSizes:
    experts: int                      # experts with matrices
    identity: int                     # router outputs after them that hand the token's own row on
    top: int
    ff: int                           # width of one expert
    groups: int = 1                   # the router's outputs form this many equal groups of neighbours
    keep: int = 1                     # of which the best `keep` can be chosen from
    shared_ff: Optional[int] = None   # width of the expert every token uses; None: there is none

    def to_dict(self) -> dict:
        out = {"kind": "moe", "expert": {"ff": self.ff},
               "router": {"experts": self.experts, "top": self.top, "identity": self.identity,
                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _read_mlp(entry: dict, where: str):
    if entry.get("mlp") is None:
        return None
    mlp = _section(entry, "mlp", where)
    kind = mlp.get("kind")
    if kind == "dense":
        return DenseSizes(whole(mlp.get("ff"), where + ".mlp.ff", 1))
    if kind == "moe":
        expert, router = _section(mlp, "expert", where + ".mlp"), _section(mlp, "router", where + ".mlp")
        experts = whole(router.get("experts"), where + ".mlp.router.experts", 1)
        identity = whole(router.get("identity", 0), where + ".mlp.router.identity", 0)
        top = whole(router.get("top"), where + ".mlp.router.top", 1)
        groups, keep = 1, 1
        if router.get("groups") is not None:
            g = _section(router, "groups", where + ".mlp.router")
            groups = whole(g.get("count", 1), where + ".mlp.router.groups.count", 1)
            keep = whole(g.get("keep", groups), where + ".mlp.router.groups.keep", 1)
        outs = experts + identity
        if outs % groups or keep > groups:
            raise ConfigError(f"{where}.mlp.router: {outs} outputs in {groups} groups of which {keep} stay")
        if top > keep * (outs // groups):
            raise ConfigError(f"{where}.mlp.router: the {top} best of the {keep * (outs // groups)} outputs of {keep} groups")
        shared = None
        if mlp.get("shared") is not None:
            shared = whole(_section(mlp, "shared", where + ".mlp").get("ff"), where + ".mlp.shared.ff", 1)
        return GroupedExpertsSizes(experts, identity, top, whole(expert.get("ff"), where + ".mlp.expert.ff", 1), groups, keep,
                                   shared)
    raise UnsupportedError(f"{where}: feed-forward kind {kind!r} is neither 'dense' nor 'moe'")


@dataclass(frozen=True)
class ZakelornLayer:
    type: str                                     # "parallel"
    mixer: ParallelSizes
    mlp: object = None                            # DenseSizes, GroupedExpertsSizes or None: the layer has no feed-forward

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class ZakelornConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: tuple = ()
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    max_positions: int = DEFAULT_MAX_POSITIONS

    ARCHITECTURE: ClassVar[str] = "Zakelorn"
    MODEL_TYPE: ClassVar[str] = "zakelorn"
    REQUIRED: ClassVar[tuple[str, ...]] = ("vocab", "width", "layers", "norm")

    @classmethod
    def from_dict(cls, raw: dict) -> "ZakelornConfig":
        cls.require(raw)
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config key 'layers' must be a list of at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or entry.get("type") != "parallel":
                kind = entry.get("type") if isinstance(entry, dict) else entry
                raise UnsupportedError(f"{where}: mixer type {kind!r} is not 'parallel'")
            layers.append(ZakelornLayer("parallel", ParallelSizes.read(_section(entry, "mixer", where), where + ".mixer"),
                                        _read_mlp(entry, where)))
        scale = 1.0
        if raw.get("embedding") is not None:
            scale = f32(_section(raw, "embedding", "config.json").get("scale", 1.0), "embedding.scale")
        cfg = cls(vocab=whole(raw["vocab"], "vocab", 1), width=whole(raw["width"], "width", 1), layers=tuple(layers),
                  norm_eps=f32(_section(raw, "norm", "config.json").get("eps"), "norm.eps"), embedding_scale=scale,
                  max_positions=whole(raw.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions", 1))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"norm.eps {self.norm_eps} must not be negative")
        for i, layer in enumerate(self.layers):
            for d in layer.mixer.right.decay:
                if not 0.0 <= d <= 1.0:
                    raise ConfigError(f"layers[{i}].mixer.right.decay {d} must lie between 0 and 1")

    def to_dict(self) -> dict:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out
