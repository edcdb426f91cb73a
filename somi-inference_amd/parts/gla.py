"""Gated linear attention: a recurrent mixer with a matrix state of fixed size per request and head.

With q, k (``heads x key_dim``) and v (``heads x value_dim``) projected from the input h and a decay per key channel,

    alpha_t = sigmoid(W2 (W1 h_t) + b)^(1 / tau)              (a low-rank projection; heads x key_dim values in (0, 1))
    S_t     = diag(alpha_t) S_(t-1) + k_t v_t^T                (per head; S: key_dim x value_dim, from zero)
    o_t     = S_t^T (q_t * key_dim^(-1/2))

each head's o is RMS-normed over its value channels with one weight shared by the heads, the heads are concatenated,
gated by ``silu(Wg h)`` and projected by Wo.  The state lives in float32 in the request's state slot and is carried
from step to step; decays, the recurrence and the norm are float32 in both engines.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import ANY_SIZE, MATRIX, VECTOR, Init, WeightSpec
from .base import Fetch, FixedStateSpec, LayerCache, Mixer, Runtime
from .linear import Projection

class GatedLinearAttention(Mixer):
    graph_safe = True
    takes_normed_rows = True      # x only goes through the stacked input projection

    ROLES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "g": "g_proj", "o": "o_proj", "norm": "o_norm",
             "a1": "decay_down", "a2": "decay_up", "a2_bias": "decay_up.bias"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, tau: float,
                 eps: float, rank: int | None = None, names: dict[str, str] | None = None,
                 suffix: str = "weight") -> None:
        """``rank``: the width of the decay's low-rank projection; None takes it from the checkpoint's tensors.
        ``names``: role -> the checkpoint's name under the prefix (``a2_bias`` and ``norm`` are whole names, the others
        are followed by ``suffix`` unless it is empty)."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.tau, self.eps = float(tau), float(eps)
        if not self.tau > 0.0:
            raise ValueError(f"{prefix}: tau must be > 0, got {tau}")
        self.rank = int(rank) if rank else None

    # ------------------------------------------------------------------ weights
    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def weight_specs(self) -> list[WeightSpec]:
        qk, vv, rank = self.num_heads * self.key_dim, self.num_heads * self.value_dim, self.rank or ANY_SIZE
        return [
            WeightSpec(self._matrix("q"), (qk, self.hidden_size), MATRIX),
            WeightSpec(self._matrix("k"), (qk, self.hidden_size), MATRIX),
            WeightSpec(self._matrix("v"), (vv, self.hidden_size), MATRIX),
            WeightSpec(self._matrix("g"), (vv, self.hidden_size), MATRIX),
            WeightSpec(self._matrix("o"), (self.hidden_size, vv), MATRIX),
            WeightSpec(self.name(self.names["norm"]), (self.value_dim,), VECTOR, Init(1.0, 0.1)),
            WeightSpec(self._matrix("a1"), (rank, self.hidden_size), MATRIX),
            WeightSpec(self._matrix("a2"), (qk, rank), MATRIX, Init(0.0, 0.5)),
            WeightSpec(self.name(self.names["a2_bias"]), (qk,), VECTOR, Init(1.0, 1.0)),
        ]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        a1, self.a2 = fetch(self._matrix("a1")), fetch(self._matrix("a2"))
        if a1.shape[0] != self.a2.shape[1]:
            raise ValueError(f"{self.prefix}: the decay's two matrices disagree about its rank "
                             f"({a1.shape[0]} and {self.a2.shape[1]})")
        self.rank = int(a1.shape[0])
        self.inputs = Projection.stacked([fetch(self._matrix(role)) for role in ("q", "k", "v", "g")] + [a1],
                                         label="q/k/v/g/decay")
        self.out = Projection(fetch(self._matrix("o")), label="o")
        self.norm_weight = fetch(self.name(self.names["norm"]))
        self.a2_bias = fetch(self.name(self.names["a2_bias"]))

    def flops(self, tokens: int, attended: int) -> float:
        """The projections, and per token and head the state's update and its product with q (two operations each on
        key_dim x value_dim elements)."""
        recurrence = 4.0 * self.num_heads * self.key_dim * self.value_dim * tokens
        decay = 2.0 * tokens * self.num_heads * self.key_dim * (self.rank or 0)
        return self.inputs.flops(tokens) + self.out.flops(tokens) + recurrence + decay

    # -------------------------------------------------------------------- cache
    def cache_spec(self) -> FixedStateSpec:
        return FixedStateSpec((self.num_heads, self.key_dim, self.value_dim), torch.float32)

    # ------------------------------------------------------------------ forward
    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or cache.state is None:
            raise ValueError(f"{self.prefix}: gated linear attention needs a state slot per request")
        qk, vv = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        rows = self.inputs(x)                                  # [N, q | k | v | g | decay]
        q, k = rows[:, :qk], rows[:, qk:2 * qk]
        v, g = rows[:, 2 * qk:2 * qk + vv], rows[:, 2 * qk + vv:2 * qk + 2 * vv]
        with stage("decays"):
            # the second matrix of the decay's projection (float32 sums and bias), then sigmoid^(1/tau) in float32
            z = linear_kernels.linear(rows[:, 2 * qk + 2 * vv:].contiguous(), self.a2, self.a2_bias, torch.float32)
            alpha = ops.gla_alpha_(z, self.tau)
        with stage("recurrence"):
            o = ops.gla_scan(q, k, v, alpha, step.entry_start, step.state_slots, cache.state, self.key_dim ** -0.5)
        with stage("norm, gate"):
            y = ops.gla_norm_gate(o, self.norm_weight, g, self.eps)
        return self.out.deferred(y)
