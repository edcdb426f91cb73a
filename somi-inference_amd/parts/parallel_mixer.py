"""Two mixers side by side: both read the same input, and the result is half the sum of their outputs, each first
RMS-normed over the model width with a weight of its own.

The two may be any registered mixers (here windowed attention beside a recurrent mixer); what they keep per request
is handed to the cache manager as one composite spec, and each gets its own part of the layer's cache back.
"""

from __future__ import annotations

import math

from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import CompositeSpec, Fetch, LayerCache, Mixer, PartSpec, Runtime
from .registry import build_part


class ParallelMixers(Mixer):
    """y = (rms_norm(left(x)) * w_left + rms_norm(right(x)) * w_right) / 2, float32.  ``names``: the sub-prefixes of the
    two mixers (``left``, ``right``) and what follows them for the norms' weights (``out``)."""

    DEFAULT_NAMES = {"left": "left", "right": "right", "out": "out"}

    def __init__(self, prefix: str, hidden_size: int, left: PartSpec, right: PartSpec, eps: float,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        self.names = {**self.DEFAULT_NAMES, **(names or {})}
        self.hidden_size, self.eps = int(hidden_size), float(eps)
        self.left = build_part("mixer", left, prefix=self.name(self.names["left"]))
        self.right = build_part("mixer", right, prefix=self.name(self.names["right"]))
        self.graph_safe = bool(self.left.graph_safe and self.right.graph_safe)
        self.portion_granule = math.lcm(int(self.left.portion_granule), int(self.right.portion_granule))
        splits = {m.entry_split for m in (self.left, self.right) if m.entry_split is not None}
        if len(splits) > 1:
            raise ValueError(f"{prefix}: the two mixers cut a step's entries at different lengths {sorted(splits)}")
        self.entry_split = splits.pop() if splits else None

    def _out(self, side: str) -> str:
        return self.name(f"{self.names[side]}.{self.names['out']}")

    def weight_specs(self) -> list[WeightSpec]:
        return (self.left.weight_specs() + self.right.weight_specs()
                + [WeightSpec(self._out(side), (self.hidden_size,), VECTOR, Init(1.0, 0.1)) for side in ("left", "right")])

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.left.load(fetch, runtime)
        self.right.load(fetch, runtime)
        self.left_weight, self.right_weight = fetch(self._out("left")), fetch(self._out("right"))

    def flops(self, tokens: int, attended: int) -> float:
        return self.left.flops(tokens, attended) + self.right.flops(tokens, attended)

    def cache_spec(self) -> CompositeSpec | None:
        parts = tuple((side, spec) for side, spec in (("left", self.left.cache_spec()), ("right", self.right.cache_spec()))
                      if spec is not None)
        return CompositeSpec(parts) if parts else None

    def forward(self, x, step, cache: LayerCache | None):
        children = cache.children if cache is not None else {}
        left = self.left.forward(x, step, children.get("left"))
        right = self.right.forward(x, step, children.get("right"))
        left, right = (y.materialize() if hasattr(y, "materialize") else y for y in (left, right))
        with stage("norms of the two mixers, mean"):
            return ops.normed_pair_mean(left, right, self.left_weight, self.right_weight, self.eps)
