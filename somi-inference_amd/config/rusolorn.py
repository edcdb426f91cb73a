"""Typed configuration of the Rusolorn decoder: parallel layers whose mixer is windowed attention beside a gated delta
rule, with a mixture of experts as feed-forward and a per-layer token input.

config.json keys: ``architecture`` ("Rusolorn"), ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``residual_mult``, ``token_side.dim`` (absent: no per-layer token input) and ``layers``, a list with one object per
layer: ``type`` ("parallel"), ``mixer`` with the two mixers' sizes under ``left`` and ``right``, and ``mlp``
(``{"kind": "moe", ...}`` or null for a layer without a feed-forward).

``mixer.left`` (attention whose values are its keys): ``heads``, ``kv_heads`` (default: ``heads``), ``dim``, ``vdim``
(the keys serve as values, so it equals ``dim``), ``scale`` (default ``dim^-1/2``), ``mask.size`` (the window).
``mixer.right`` (gated delta rule): ``heads``, ``kv_heads`` (q/k heads; default ``heads``), ``dim``, ``vdim``, ``conv``
(taps of the short convolution).  ``mlp``: ``router`` (``experts``, ``top``, optional ``groups`` with ``count`` and
``keep``), ``expert`` (``ff``, ``limit``) and optionally ``shared`` (``ff``, ``limit``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class RusolornAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "RusolornAttention":
        mask = keys.sub("mask")
        if mask is None:
            raise ConfigError(f"{where}: required key 'mask' is missing")
        heads, dim = keys.integer("heads", minimum=1), keys.integer("dim", minimum=1)
        out = cls(heads=heads, kv_heads=keys.integer("kv_heads", heads, minimum=1), dim=dim,
                  vdim=keys.integer("vdim", dim, minimum=1), scale=keys.number("scale", dim ** -0.5),
                  window=mask.integer("size", minimum=1))
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.heads % self.kv_heads:
            raise ConfigError(f"{where}: 'heads' ({self.heads}) must be divisible by 'kv_heads' ({self.kv_heads})")
        if self.vdim != self.dim:
            raise ConfigError(f"{where}: the values are the keys, so 'vdim' ({self.vdim}) must equal 'dim' ({self.dim})")

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "mask": {"size": self.window}}


@dataclass(frozen=True)
class RusolornDeltaRule:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "RusolornDeltaRule":
        heads = keys.integer("heads", minimum=1)
        out = cls(heads=heads, kv_heads=keys.integer("kv_heads", heads, minimum=1), dim=keys.integer("dim", minimum=1),
                  vdim=keys.integer("vdim", minimum=1), conv=keys.integer("conv", minimum=1))
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.heads % self.kv_heads:
            raise ConfigError(f"{where}: 'heads' ({self.heads}) must be divisible by 'kv_heads' ({self.kv_heads})")

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class RusolornExperts:
    experts: int
    top: int
    ff: int
    limit: float
    groups: int = 1
    keep: int = 1
    shared_ff: int | None = None
    shared_limit: float | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "RusolornExperts":
        if keys.string("kind", "moe") != "moe":
            raise ConfigError(f"{where}: 'kind' must be 'moe', got {keys.string('kind')!r}")
        router, expert, shared = keys.sub("router"), keys.sub("expert"), keys.sub("shared")
        if router is None or expert is None:
            raise ConfigError(f"{where}: a mixture of experts needs 'router' and 'expert'")
        groups = router.sub("groups")
        out = cls(experts=router.integer("experts", minimum=1), top=router.integer("top", minimum=1),
                  ff=expert.integer("ff", minimum=1), limit=expert.number("limit", positive=True),
                  groups=groups.integer("count", minimum=1) if groups else 1,
                  keep=groups.integer("keep", minimum=1) if groups else 1,
                  shared_ff=shared.integer("ff", minimum=1) if shared else None,
                  shared_limit=shared.number("limit", positive=True) if shared else None)
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.experts % self.groups or self.keep > self.groups:
            raise ConfigError(f"{where}: 'groups' (count {self.groups}, keep {self.keep}) must divide the {self.experts} experts")
        if self.top > self.keep * (self.experts // self.groups):
            raise ConfigError(f"{where}: 'top' ({self.top}) is more than the experts of the kept groups")

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                               "router": {"experts": self.experts, "top": self.top,
                                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass(frozen=True)
class RusolornLayer:
    left: RusolornAttention
    right: RusolornDeltaRule
    mlp: RusolornExperts | None = None
    type: str = "parallel"

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": {"left": self.left.to_dict(), "right": self.right.to_dict()},
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class RusolornConfig(ModelConfig):
    architecture: ClassVar[str] = "Rusolorn"

    vocab: int
    width: int
    layers: tuple[RusolornLayer, ...]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    residual_mult: float = 1.0
    token_side_dim: int | None = None

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: 'vocab' and 'width' must be >= 1 and 'layers' must not be empty")
        object.__setattr__(self, "layers", tuple(self.layers))
        for index, layer in enumerate(self.layers):
            where = f"config.json:layers[{index}]"
            if layer.type != "parallel":
                raise ConfigError(f"{where}: 'type' must be 'parallel', got {layer.type!r}")
            layer.left.check(where + ":mixer:left")
            layer.right.check(where + ":mixer:right")
            if layer.mlp is not None:
                layer.mlp.check(where + ":mlp")

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "RusolornConfig":
        keys = KeyReader(data)
        raw_layers = keys.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for index, raw in enumerate(raw_layers):
            where = f"config.json:layers[{index}]"
            layer = KeyReader(raw, where)
            kind = layer.string("type")
            if kind != "parallel":
                raise ConfigError(f"{where}: 'type' must be 'parallel', got {kind!r}")
            mixer = layer.sub("mixer")
            if mixer is None or mixer.sub("left") is None or mixer.sub("right") is None:
                raise ConfigError(f"{where}: 'mixer' needs 'left' and 'right'")
            mlp = layer.sub("mlp")
            layers.append(RusolornLayer(
                left=RusolornAttention.read(mixer.sub("left"), where + ":mixer:left"),
                right=RusolornDeltaRule.read(mixer.sub("right"), where + ":mixer:right"),
                mlp=None if mlp is None else RusolornExperts.read(mlp, where + ":mlp"), type=kind))
        norm, embedding, side = keys.sub("norm"), keys.sub("embedding"), keys.sub("token_side")
        return cls(vocab=keys.integer("vocab", minimum=1), width=keys.integer("width", minimum=1), layers=tuple(layers),
                   norm_eps=norm.number("eps", 1e-6, positive=True) if norm else 1e-6,
                   embedding_scale=embedding.number("scale", 1.0) if embedding else 1.0,
                   residual_mult=keys.number("residual_mult", 1.0),
                   token_side_dim=side.integer("dim", minimum=1) if side else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                               "residual_mult": self.residual_mult, "layers": [layer.to_dict() for layer in self.layers]}
        if self.token_side_dim is not None:
            out["token_side"] = {"dim": self.token_side_dim}
        return out
