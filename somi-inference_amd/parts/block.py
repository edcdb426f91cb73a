"""Arrangements of a layer's parts around the residual stream."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
from .base import Block, LayerCache, Part, PartSpec
from .registry import build_part
from .residual import ResidualStream


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h)).

    Reference: somi_inference/models/qwen2.py:325-339.  ``names`` gives the
    sub-prefixes of the four parts under the layer's prefix (an empty one puts a
    part's tensors directly under the layer's).  A layer without a feed-forward
    (``feed_forward=None``) has the first sublayer only.
    """
    graph_safe = True

    DEFAULT_NAMES = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                     "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, mixer_norm: PartSpec,
                 ffn_norm: PartSpec | None = None, names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.mixer_norm = build_part("norm", mixer_norm, prefix=self.name(sub["mixer_norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.ffn_norm = self.feed_forward = None
        if feed_forward is not None:
            if ffn_norm is None:
                raise ValueError(f"{prefix}: a feed-forward needs its norm")
            self.ffn_norm = build_part("norm", ffn_norm, prefix=self.name(sub["ffn_norm"]))
            self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))

    def parts(self) -> list[Part]:
        parts = [self.mixer_norm, self.mixer]
        return parts + [self.ffn_norm, self.feed_forward] if self.feed_forward is not None else parts

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        x = stream.normed(self.mixer_norm, lazy=getattr(self.mixer, "takes_normed_rows", False))
        stream.add(self.mixer.forward(x, step, cache))
        if self.feed_forward is None:
            return
        x = stream.normed(self.ffn_norm, lazy=getattr(self.feed_forward, "takes_normed_rows", False))
        stream.add(self.feed_forward.forward(x, step))


class ParallelBlock(Block):
    """One norm, and mixer and feed-forward side by side: with x' = norm(h), ``h += mult * (mixer(x') + ff(x'))``;
    then, if the layer has one, a per-layer token input adds to h from the token itself (``token_input``, a part of
    the category of that name with ``add_to(h, x, step, mult)``).  The sum is float32; a layer without a feed-forward
    adds the mixer alone.  ``names``: the sub-prefixes of the norm, the mixer, the feed-forward and the token input."""

    DEFAULT_NAMES = {"norm": "input_layernorm", "mixer": "self_attn", "feed_forward": "mlp", "token_input": "token_input"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, norm: PartSpec,
                 residual_mult: float = 1.0, token_input: PartSpec | None = None,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.residual_mult = float(residual_mult)
        self.norm = build_part("norm", norm, prefix=self.name(sub["norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.feed_forward = (build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))
                             if feed_forward is not None else None)
        self.token_input = (build_part("token_input", token_input, prefix=self.name(sub["token_input"]))
                            if token_input is not None else None)
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts())

    def parts(self) -> list[Part]:
        return [part for part in (self.norm, self.mixer, self.feed_forward, self.token_input) if part is not None]

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        x = stream.normed(self.norm)
        mixed = _float32_rows(self.mixer.forward(x, step, cache))
        fed = _float32_rows(self.feed_forward.forward(x, step)) if self.feed_forward is not None else None
        h = stream.settle()
        with stage("residual add"):
            copy = ops.scaled_add(h, mixed, fed, self.residual_mult,
                                  self.runtime.dtype if self.token_input is not None else None)
        if self.token_input is not None:
            self.token_input.add_to(h, copy, step, self.residual_mult)


def _float32_rows(y):
    """A sublayer's output as float32 rows (a promised product is computed, 16-bit rows are widened)."""
    if hasattr(y, "materialize"):
        y = y.materialize()
    return y if y.dtype == torch.float32 else y.to(torch.float32)
