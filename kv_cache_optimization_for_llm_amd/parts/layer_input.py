"""What a layer adds to the residual stream from outside the stream: the token's own row of a table.

:class:`GatedTableInput` (``"gated_table"``): a second embedding table holds, for every token id, a
row of ``layers * dim`` values; layer i takes its ``dim`` columns ``e``, multiplies them by a gate
computed from the stream, ``act(W_gate x) * e``, and projects the product back to the stream's width,
``y = W_proj (act(W_gate x) * e)``.  ``y`` enters the stream under an RMS norm with a plain weight
(``x += y / sqrt(mean(y^2) + eps) * w``): the part is its own norm for the block arrangement
(:meth:`into_stream`).  The table is one tensor shared by all layers.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import LAYER_INPUTS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import MixerContext, Part
from .linear import Linear


@LAYER_INPUTS.register("gated_table")
class GatedTableInput(Part):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, dim: int, table_name: str, table_rows: int, table_width: int,
                 column: int, eps: float, activation: str = "gelu_tanh", tensor_names: Optional[Dict[str, str]] = None):
        """``table_name``: the table's full tensor name (no prefix: every layer names the same one), ``[table_rows,
        table_width]``; this layer's columns are ``column .. column + dim``.  ``tensor_names`` maps ``gate``,
        ``proj`` and ``norm`` to names behind ``prefix``."""
        super().__init__(prefix)
        if activation not in K.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(K.ACTIVATIONS)}")
        self.hidden_size, self.dim, self.eps, self.activation = int(hidden_size), int(dim), float(eps), activation
        self.table_name, self.table_rows, self.table_width, self.column = table_name, int(table_rows), int(table_width), int(column)
        if not 0 <= self.column <= self.table_width - self.dim:
            raise ValueError(f"{prefix}: columns {column}..{column + dim} lie outside a table row of {table_width}")
        names = dict(gate="gate", proj="proj", norm="norm")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        return {self.table_name: TensorSpec((self.table_rows, self.table_width)),
                n["gate"]: TensorSpec((self.dim, self.hidden_size)), n["proj"]: TensorSpec((self.hidden_size, self.dim)),
                n["norm"]: TensorSpec((self.hidden_size,), init="norm", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.table_name]
        self.gate, self.proj = Linear(tensors[self.names["gate"]]), Linear(tensors[self.names["proj"]])
        self.weight = tensors[self.names["norm"]].contiguous()

    def activation_elements(self) -> int:
        return 2 * self.dim + self.hidden_size

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        batch = ctx.batch
        z = self.gate(x)
        g = K.table_gate(z, self.table, batch.token_ids, self.column, torch.empty_like(z), self.activation,
                         getattr(batch, "feedback", None))
        return self.proj(g)

    def into_stream(self, stream: torch.Tensor, y: torch.Tensor, copy: Optional[torch.Tensor] = None) -> None:
        K.norm_into_stream(stream, y, self.weight, self.eps, copy)
