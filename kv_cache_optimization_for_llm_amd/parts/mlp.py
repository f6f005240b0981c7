"""Gated feed-forward: ``down( act(gate(x)) * up(x) )``, no biases; SwiGLU is ``act = silu``
(reference: ``base/src/engine.cu:780-858``, ``siluKernel`` ``base/src/kernels.cu:45-52``).

Gate and up matrices are joined at load time into one ``[2 * intermediate, hidden]`` matrix.
The activation is a parameter (``silu``, ``relu``, ``gelu_tanh``); the products that apply it in
their epilogue exist for ``silu``, another activation runs as its own kernel behind the joined
product.  ``"none"`` is the feed-forward of a layer that has none.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import BranchTail, FeedForward, MixerContext, NormedRows
from .linear import Linear


@FEED_FORWARDS.register("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward branch: the block skips it."""

    graph_safe = True
    absent = True

    def __init__(self, prefix: str = "", **_ignored):
        super().__init__(prefix)

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        raise RuntimeError("a layer without a feed-forward has no branch to run")


@FEED_FORWARDS.register("gated")
@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 limit: float = 0.0, tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``gate``, ``up``, ``down`` to the matrices' names behind ``prefix``.
        ``activation="swish_clamped"`` with its ``limit``: ``g sigmoid(1.702 g) (u + 1)`` with ``g = min(gate,
        limit)``, ``u = clamp(up, -limit, limit)``."""
        super().__init__(prefix)
        if activation not in K.GATED_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(K.GATED_ACTIVATIONS)}")
        self.activation, self.limit = activation, float(limit)
        names = dict(gate="gate_proj.weight", up="up_proj.weight", down="down_proj.weight")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, h, i = self.names, self.hidden_size, self.intermediate_size
        return {n["gate"]: TensorSpec((i, h)), n["up"]: TensorSpec((i, h)), n["down"]: TensorSpec((h, i))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            raise ValueError(f"{p}: gate and up projection weights are stored in different dtypes")
        # (the tiled copy of a joined matrix pairs gate and up rows for the products that activate in their
        # epilogue; an activation that runs as its own kernel reads the plain product's two halves)
        self.gate_up = Linear(torch.cat([g, u], dim=0), halves=2 if self.activation in K.ACTIVATIONS else 1)
        self.down = Linear(tensors[self.names["down"]])

    fuses_tail = True

    def activation_elements(self) -> int:
        # gate and up, their gated product, the down projection
        return 3 * self.intermediate_size + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        """``x`` may be NormedRows; with a ``tail`` the down projection adds into the residual
        stream and prepares the next norm when the shapes allow (NormedRows are returned)."""
        rows = x.shape[0]
        # (the products' epilogues know the plain activations; a clamped one runs as its own kernel)
        up_kernel = self.gate_up.fused_kernel(rows, x.dtype) if self.activation in K.ACTIVATIONS else None
        # Both products in their few-rows form and at most 16 rows: the activations go from one to
        # the other in the order the second one's lanes read them (ops.kernels.TiledRows).
        tiled = (up_kernel == Linear.FEW_ROWS and rows <= K.TiledRows.MAX_ROWS and self.intermediate_size % 8 == 0
                 and self.down.residual_kernel(rows, x.dtype, tail) == Linear.FEW_ROWS)
        if tiled:
            act = K.TiledRows(rows, self.intermediate_size, x.device)
        else:
            act = torch.empty((rows, self.intermediate_size), dtype=x.dtype, device=x.device)
        if up_kernel is not None:
            # activation fused into the product; an unfinished input norm is finished there too
            self.gate_up.gated(x, act, self.activation)
        elif self.activation == "silu":
            K.silu_mul(self.gate_up(x), act)
        else:
            K.act_mul(self.gate_up(x), act, self.activation, self.limit)
        if tail is not None:
            fused = self.down.into_residual(act, tail)
            if fused is not None:
                return fused
        if tiled:
            act = act.to_rows()
        return self.down(act)


@FEED_FORWARDS.register("mlp")
class PlainMLP(FeedForward):
    """A feed-forward that is not gated: ``down(act(up(x)))`` without biases; ``act`` one of silu, relu,
    gelu_tanh, applied by its own kernel between the two products."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh",
                 tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``up``, ``down`` to the matrices' names behind ``prefix``."""
        super().__init__(prefix)
        if activation not in K.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(K.ACTIVATIONS)}")
        self.activation = activation
        names = dict(up="up", down="down")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, h, i = self.names, self.hidden_size, self.intermediate_size
        return {n["up"]: TensorSpec((i, h)), n["down"]: TensorSpec((h, i))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.up, self.down = Linear(tensors[self.names["up"]]), Linear(tensors[self.names["down"]])

    def activation_elements(self) -> int:
        return 2 * self.intermediate_size + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        z = self.up(x)
        return self.down(K.bias_act(z, z, self.activation))
