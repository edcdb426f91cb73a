"""The gated delta rule: a recurrent mixer whose matrix state forgets by a decay and learns by an error.

With q, k (``groups`` heads of ``key_dim``) and v (``heads`` heads of ``value_dim``; head h reads q/k head
``h // (heads / groups)``) projected from the input x, each channel passed through a short causal convolution over
time (``taps`` wide, the last tap on the current token, zeros before a sequence's start) and SiLU, q and k then
scaled to unit length per head (``x / sqrt(sum x^2 + 1e-6)``) and q by ``key_dim^-1/2``,

    beta_t = sigmoid(W_b x_t)                                       (per head)
    g_t    = exp(-exp(A_log) * softplus(W_a x_t + dt_bias))         (per head, in (0, 1))
    S     <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t

per head (S: key_dim x value_dim, from zero), so that o_t sees the token's own write.  Each head's o is RMS-normed
over its value channels with one weight shared by the heads, gated by ``silu(W_g x)`` and projected by W_o.  A
request's S and the convolution's last ``taps - 1`` inputs live in float32 in its state slot and are carried from
step to step; the convolution, the unit norms, beta, the decay, the recurrence and the norm are float32 in both
engines.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import CompositeSpec, Fetch, FixedStateSpec, LayerCache, Mixer, Runtime
from .linear import Projection


class GatedDeltaRule(Mixer):
    graph_safe = True

    ROLES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "g": "g_proj", "o": "o_proj", "b": "b_proj", "a": "a_proj",
             "norm": "o_norm", "a_log": "A_log", "dt_bias": "dt_bias", "conv": "conv"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_groups: int, key_dim: int, value_dim: int,
                 taps: int, eps: float, names: dict[str, str] | None = None, suffix: str = "weight") -> None:
        """``names``: role -> the checkpoint's name under the prefix (``norm``, ``a_log`` and ``dt_bias`` are whole
        names; ``conv`` is what follows a projection's name for its taps, ``<q>.<conv>``; the others are followed by
        ``suffix`` unless it is empty)."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        if num_heads % num_groups != 0:
            raise ValueError(f"{prefix}: heads ({num_heads}) must be divisible by the q/k heads ({num_groups})")
        if not 1 <= int(taps) <= ops.DELTA_MAX_TAPS:
            raise ValueError(f"{prefix}: a convolution of {taps} taps; 1 to {ops.DELTA_MAX_TAPS} are supported")
        self.hidden_size, self.num_heads, self.num_groups = int(hidden_size), int(num_heads), int(num_groups)
        self.key_dim, self.value_dim, self.taps, self.eps = int(key_dim), int(value_dim), int(taps), float(eps)

    # ------------------------------------------------------------------ weights
    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def _taps(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.names['conv']}")

    def weight_specs(self) -> list[WeightSpec]:
        qk, vv, h = self.num_groups * self.key_dim, self.num_heads * self.value_dim, self.hidden_size
        return [
            WeightSpec(self._matrix("q"), (qk, h), MATRIX), WeightSpec(self._taps("q"), (qk, self.taps), VECTOR, Init(0.3, 0.3)),
            WeightSpec(self._matrix("k"), (qk, h), MATRIX), WeightSpec(self._taps("k"), (qk, self.taps), VECTOR, Init(0.3, 0.3)),
            WeightSpec(self._matrix("v"), (vv, h), MATRIX), WeightSpec(self._taps("v"), (vv, self.taps), VECTOR, Init(0.3, 0.3)),
            WeightSpec(self._matrix("b"), (self.num_heads, h), MATRIX),
            WeightSpec(self._matrix("a"), (self.num_heads, h), MATRIX),
            WeightSpec(self.name(self.names["a_log"]), (self.num_heads,), VECTOR, Init(-1.0, 0.5)),
            WeightSpec(self.name(self.names["dt_bias"]), (self.num_heads,), VECTOR, Init(0.0, 0.5)),
            WeightSpec(self.name(self.names["norm"]), (self.value_dim,), VECTOR, Init(1.0, 0.1)),
            WeightSpec(self._matrix("g"), (vv, h), MATRIX),
            WeightSpec(self._matrix("o"), (h, vv), MATRIX),
        ]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.inputs = Projection.stacked([fetch(self._matrix(role)) for role in ("q", "k", "v", "g")], label="q/k/v/g")
        # beta's and the decay's projections leave their product in float32: a few rows of the matrix
        self.rates = Projection.stacked([fetch(self._matrix(role)) for role in ("b", "a")], label="beta/decay")
        self.out = Projection(fetch(self._matrix("o")), label="o")
        self.conv_taps = torch.cat([fetch(self._taps(role)) for role in ("q", "k", "v")], dim=0).contiguous()
        self.a_log, self.dt_bias = fetch(self.name(self.names["a_log"])), fetch(self.name(self.names["dt_bias"]))
        self.norm_weight = fetch(self.name(self.names["norm"]))

    def flops(self, tokens: int, attended: int) -> float:
        """The projections, and per token and head three passes over the state (its products with k and q, its update)."""
        recurrence = 6.0 * self.num_heads * self.key_dim * self.value_dim * tokens
        return self.inputs.flops(tokens) + self.rates.flops(tokens) + self.out.flops(tokens) + recurrence

    # -------------------------------------------------------------------- cache
    @property
    def channels(self) -> int:
        return 2 * self.num_groups * self.key_dim + self.num_heads * self.value_dim

    def cache_spec(self) -> CompositeSpec:
        return CompositeSpec((
            ("state", FixedStateSpec((self.num_heads, self.key_dim, self.value_dim), torch.float32)),
            ("conv", FixedStateSpec((max(self.taps - 1, 1), self.channels), torch.float32)),
        ))

    # ------------------------------------------------------------------ forward
    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or "state" not in cache.children or "conv" not in cache.children:
            raise ValueError(f"{self.prefix}: the gated delta rule needs a state slot per request")
        state, conv = cache.children["state"].state, cache.children["conv"].state
        vv = self.num_heads * self.value_dim
        if hasattr(x, "materialize"):
            x = x.materialize()
        rows = self.inputs(x)                                  # [N, q | k | v | g]
        with stage("beta, decay"):
            ab = linear_kernels.linear(x, self.rates.weight, None, torch.float32)
        with stage("convolution, unit norms"):
            qkv, beta, decay = ops.delta_prepare(rows, ab, self.conv_taps, conv, step, self.a_log, self.dt_bias,
                                                 self.num_groups, self.num_heads, self.key_dim, self.value_dim)
        with stage("recurrence"):
            o = ops.delta_scan(qkv, beta, decay, step.entry_start, step.state_slots, state, self.num_groups)
        with stage("norm, gate"):
            y = ops.gla_norm_gate(o, self.norm_weight, rows[:, self.channels:self.channels + vv], self.eps)
        return self.out.deferred(y)
