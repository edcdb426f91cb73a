"""Typed configuration of the Kamedra decoder: a stack of layers, each with one of two mixers.

config.json keys: ``architecture`` ("Kamedra"), ``vocab``, ``width``, ``norm.eps``, ``logit_softcap`` and ``layers``, a
list with one object per layer: ``type`` ("attention" or "gla"), ``mixer`` (the mixer's sizes and constants) and
``mlp`` (``{"kind": "dense", "ff": ...}`` or null for a layer without a feed-forward).

An attention mixer gives ``heads``, ``kv_heads`` (default: ``heads``), ``dim`` (query/key size of one map), ``vdim``
(default: ``dim``), ``scale`` (default: ``dim^-1/2``), ``diff``,
``mask`` (``size``, ``keep_first``), ``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``, ``low``,
``high``, ``original``) and optionally ``kv_from``, the index of the earlier layer whose keys and values it reads.
A gla mixer gives ``heads``, ``dim``, ``vdim`` and ``tau``; the width of its decay's low-rank projection is the
checkpoint's (``rank`` may name it, which seeded random weights need).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    low: float
    high: float
    original: int

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class KamedraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    mask_size: int
    mask_keep_first: int
    rot_base: float
    rot_dims: int
    rot_scaling: RotaryScaling | None = None
    kv_from: int | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "KamedraAttention":
        mask, rot = keys.sub("mask"), keys.sub("rot")
        if mask is None or rot is None:
            raise ConfigError(f"{where}: an attention mixer needs 'mask' and 'rot'")
        scaling = rot.sub("scaling")
        out = cls(
            heads=keys.integer("heads", minimum=1), kv_heads=keys.integer("kv_heads", keys.integer("heads", minimum=1), minimum=1),
            dim=keys.integer("dim", minimum=1), vdim=keys.integer("vdim", keys.integer("dim", minimum=1), minimum=1),
            scale=keys.number("scale", keys.integer("dim", minimum=1) ** -0.5), diff=keys.number("diff"),
            mask_size=mask.integer("size", minimum=1), mask_keep_first=mask.integer("keep_first", 0, minimum=0),
            rot_base=rot.number("base", positive=True), rot_dims=rot.integer("dims", minimum=0),
            rot_scaling=None if scaling is None else RotaryScaling(
                scaling.number("factor", positive=True), scaling.number("low"), scaling.number("high"),
                scaling.integer("original", minimum=1)),
            kv_from=keys.optional_integer("kv_from", minimum=0))
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: 'heads' ({out.heads}) must be divisible by 'kv_heads' ({out.kv_heads})")
        if out.rot_dims % 2 or out.rot_dims > out.dim:
            raise ConfigError(f"{where}: 'rot.dims' ({out.rot_dims}) must be even and at most 'dim' ({out.dim})")
        if out.rot_scaling is not None and out.rot_scaling.high == out.rot_scaling.low:
            raise ConfigError(f"{where}: 'rot.scaling.high' and 'low' must differ")
        return out

    def to_dict(self) -> dict[str, Any]:
        rot: dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "diff": self.diff,
                               "mask": {"size": self.mask_size, "keep_first": self.mask_keep_first}, "rot": rot}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class KamedraGLA:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "KamedraGLA":
        return cls(heads=keys.integer("heads", minimum=1), dim=keys.integer("dim", minimum=1),
                   vdim=keys.integer("vdim", minimum=1), tau=keys.number("tau", positive=True),
                   rank=keys.optional_integer("rank", minimum=1))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class KamedraLayer:
    type: str                                   # "attention" or "gla"
    mixer: KamedraAttention | KamedraGLA
    ff: int | None = None                       # the dense feed-forward's inner size; None: no feed-forward

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class KamedraConfig(ModelConfig):
    architecture: ClassVar[str] = "Kamedra"

    vocab: int
    width: int
    layers: tuple[KamedraLayer, ...]
    norm_eps: float = 1e-6
    logit_softcap: float | None = None

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: 'vocab' and 'width' must be >= 1 and 'layers' must not be empty")
        object.__setattr__(self, "layers", tuple(self.layers))
        for index, layer in enumerate(self.layers):
            if layer.type != "attention" or layer.mixer.kv_from is None:
                continue
            source = layer.mixer.kv_from
            if not 0 <= source < index or self.layers[source].type != "attention":
                raise ConfigError(f"config.json: layer {index}: 'kv_from' ({source}) must name an earlier attention layer")
            theirs, mine = self.layers[source].mixer, layer.mixer
            if theirs.kv_from is not None:
                raise ConfigError(f"config.json: layer {index}: layer {source} has no keys and values of its own")
            same = ("kv_heads", "dim", "vdim", "rot_base", "rot_dims", "rot_scaling")
            if any(getattr(theirs, key) != getattr(mine, key) for key in same):
                raise ConfigError(f"config.json: layer {index} reads the keys and values of layer {source}: their "
                                  f"kv_heads, dim, vdim and rot must agree")

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "KamedraConfig":
        keys = KeyReader(data)
        raw_layers = keys.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for index, raw in enumerate(raw_layers):
            where = f"config.json:layers[{index}]"
            layer = KeyReader(raw, where)
            kind = layer.string("type")
            mixer = layer.sub("mixer")
            if mixer is None:
                raise ConfigError(f"{where}: required key 'mixer' is missing")
            if kind == "attention":
                parsed: KamedraAttention | KamedraGLA = KamedraAttention.read(mixer, where + ":mixer")
            elif kind == "gla":
                parsed = KamedraGLA.read(mixer, where + ":mixer")
            else:
                raise ConfigError(f"{where}: 'type' must be 'attention' or 'gla', got {kind!r}")
            ff = None
            mlp = layer.sub("mlp")
            if mlp is not None:
                if mlp.string("kind", "dense") != "dense":
                    raise ConfigError(f"{where}:mlp: 'kind' must be 'dense', got {mlp.string('kind')!r}")
                ff = mlp.integer("ff", minimum=1)
            layers.append(KamedraLayer(kind, parsed, ff))
        norm = keys.sub("norm")
        softcap = keys.number("logit_softcap", 0.0)
        return cls(vocab=keys.integer("vocab", minimum=1), width=keys.integer("width", minimum=1),
                   layers=tuple(layers), norm_eps=norm.number("eps", 1e-6, positive=True) if norm else 1e-6,
                   logit_softcap=softcap if softcap > 0.0 else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out
