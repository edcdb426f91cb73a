"""RMSNorm.  Reference: somi_inference/models/qwen2.py:46-62."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import Fetch, Norm, Runtime


class RMSNorm(Norm):
    """y = w * x * rsqrt(mean(x^2) + eps), no mean subtraction, no bias
    (qwen2.py:55-62).  Square, mean, rsqrt and scale are float32."""
    graph_safe = True
    fusable = True        # weight * (h / sqrt(mean(h^2) + eps)): what a projection can apply while it loads h

    def __init__(self, prefix: str, hidden_size: int, eps: float,
                 init: tuple[float, float] = (1.0, 0.1), tensor: str = "weight") -> None:
        """``tensor``: what the checkpoint calls the scale under the part's prefix."""
        super().__init__(prefix)
        self.tensor = str(tensor)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self._init = Init(*init)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.name(self.tensor), (self.hidden_size,), VECTOR, self._init)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name(self.tensor))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype)

    def add_forward(self, h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype, delta=delta)


class DynamicTanh(Norm):
    """y = tanh(alpha * x) * w + b: a norm that computes no mean and no variance.  ``alpha`` is one stored number,
    ``w`` and ``b`` vectors; the tensors are ``<tensor>``, ``<tensor>.alpha`` and ``<tensor>.b`` under the prefix.
    float32 throughout, rounded once to the compute dtype."""
    graph_safe = True
    fusable = False       # not a row scale: no projection applies it while it loads its rows

    def __init__(self, prefix: str, hidden_size: int, tensor: str = "weight", alpha_init: float = 0.5) -> None:
        super().__init__(prefix)
        self.tensor = str(tensor)
        self.hidden_size = int(hidden_size)
        self.alpha_init = float(alpha_init)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        name = self.name(self.tensor)
        return [WeightSpec(name, (self.hidden_size,), VECTOR, Init(1.0, 0.1)),
                WeightSpec(f"{name}.b", (self.hidden_size,), VECTOR, Init(0.0, 0.1)),
                WeightSpec(f"{name}.alpha", (), VECTOR, Init(self.alpha_init, 0.0))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        name = self.name(self.tensor)
        self.weight, self.bias = fetch(name), fetch(f"{name}.b")
        self.alpha = fetch(f"{name}.alpha").reshape(1).contiguous()      # stays on the device: the kernel reads it

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.dynamic_tanh(h, self.weight, self.bias, self.alpha, self.runtime.dtype)
