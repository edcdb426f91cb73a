"""A per-layer token input: every layer adds something that depends on the token itself, from a second embedding
table of which each layer owns a slice of ``dim`` columns.

With x the residual stream after the layer's sublayers and e the layer's slice of the table's row of the token,

    y = W_proj (gelu_tanh(W_gate x) * e);      x <- x + mult * y / rms(y) * w

(rms with eps inside the root, a plain weight).  The table is one tensor shared by the layers.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import Fetch, Part, Runtime


class GatedTokenInput(Part):
    graph_safe = True

    ROLES = {"gate": "gate", "proj": "proj", "norm": "norm"}

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, dim: int, table: str, table_width: int,
                 offset: int, eps: float, names: dict[str, str] | None = None) -> None:
        """``table``: the full name of the shared table ``[vocab, table_width]``; this layer reads its columns
        ``offset .. offset + dim``."""
        super().__init__(prefix)
        self.names = {**self.ROLES, **(names or {})}
        self.hidden_size, self.vocab_size, self.dim = int(hidden_size), int(vocab_size), int(dim)
        self.table_name, self.table_width, self.offset, self.eps = str(table), int(table_width), int(offset), float(eps)
        if not 0 <= self.offset <= self.table_width - self.dim:
            raise ValueError(f"{prefix}: columns {offset}..{offset + dim} do not fit a table {table_width} wide")

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.table_name, (self.vocab_size, self.table_width), MATRIX),
                WeightSpec(self.name(self.names["gate"]), (self.dim, self.hidden_size), MATRIX),
                WeightSpec(self.name(self.names["proj"]), (self.hidden_size, self.dim), MATRIX),
                WeightSpec(self.name(self.names["norm"]), (self.hidden_size,), VECTOR, Init(1.0, 0.1))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        # the layers of a model share one copy of the table: it is kept with the loader's fetch function
        held = getattr(fetch, "_shared_tables", None)
        if held is None:
            held = {}
            try:
                fetch._shared_tables = held
            except AttributeError:
                pass
        if self.table_name not in held:
            held[self.table_name] = fetch(self.table_name)
        self.table = held[self.table_name]
        self.gate = fetch(self.name(self.names["gate"]))
        self.proj = fetch(self.name(self.names["proj"]))
        self.norm_weight = fetch(self.name(self.names["norm"]))

    def flops(self, tokens: int, attended: int) -> float:
        return 4.0 * tokens * self.dim * self.hidden_size

    def add_to(self, h: torch.Tensor, x: torch.Tensor, step, mult: float) -> None:
        """h: the float32 residual rows; x: the same rows in the compute dtype.  Adds the layer's token input to h."""
        with stage("token input"):
            gate = linear_kernels.linear(x, self.gate, None, x.dtype)
            gated = ops.gated_table_rows(gate, self.table, step.token_ids, self.offset)
            y = linear_kernels.linear(gated, self.proj, None, torch.float32)
            ops.normed_add(h, y, self.norm_weight, self.eps, mult)
