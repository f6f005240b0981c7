"""A routed feed-forward: every token is sent to ``top`` of ``experts`` small feed-forward layers
``W_down act(W_up x)`` and takes the weighted sum of what they return.

Router: ``scores = softmax(W_router x)`` in fp32 over all router outputs.  The ``top`` outputs with
the largest ``scores + correction`` (a stored vector that shifts the choice but not the weights)
are chosen; their weights are the plain scores (``renormalise``: divided by their sum).  The last
``identity`` router outputs stand for experts that return their input: they have no tensors.
``router_bias``: a stored vector added to the logits themselves; ``softmax_over="chosen"``: the
largest logits are chosen and the weights are the softmax over the chosen logits alone.
``gated``: an expert is ``W_down (act(W_gate x) * (W_up x))``; its gate and up matrices are stacked
row by row in turns at load time, so that one product's epilogue has both halves of every output.
``shared_intermediate``: one more expert of that width (its tensors behind ``shared.``) that every
token uses with weight 1; it runs as an ordinary gated feed-forward and is added to the sum.

Everything from the router's logits to the sum stays on the device (``csrc/moe.hip``): the chosen
(token, choice) slots are sorted by expert into tiles of 16 rows, one kernel runs the first
product of every tile with its activation, a second the other product times the slot's weight,
and a third adds a token's rows up - no count of tokens per expert reaches the host, so a step
with this layer can be captured into a graph.  The experts' matrices are stacked at load time
(``[experts, ff, hidden]`` and ``[experts, hidden, ff]``).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import FeedForward, MixerContext


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True
    # a function ``(part, idx [T, top] on the device)`` called after every routing of an eager step:
    # for whoever wants to see which experts the tokens were sent to (tests do); None: nothing is called
    on_route = None

    def __init__(self, prefix: str, *, hidden_size: int, intermediate_size: int, experts: int, top: int,
                 identity: int = 0, activation: str = "gelu", correction: bool = True, renormalise: bool = False,
                 gated: bool = False, router_bias: bool = False, softmax_over: str = "all",
                 shared_intermediate: int = 0, scores: str = "softmax", groups: int = 1, keep_groups: int = 1,
                 group_top: int = 2, weight_scale: float = 1.0, sum_eps: float = 0.0, limit: float = 0.0,
                 shared_limit: Optional[float] = None, shared_gate: bool = False,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``scores="sigmoid"``: every router output's score is its own sigmoid.  ``groups`` > 1: the outputs
        form so many equal runs of neighbours, a run's score is the sum of its ``group_top`` largest choice
        scores (score + correction), and only outputs of the ``keep_groups`` best runs can be chosen.
        ``weight_scale`` multiplies the weights; ``sum_eps`` is added to the sum they are divided by
        (``renormalise``).  ``activation="swish_clamped"`` (gated experts) with ``limit``: ``g sigmoid(1.702 g)
        (u + 1)``, ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``; ``shared_limit``: the limit of the
        expert every token uses (default: ``limit``).  ``shared_gate``: that expert's result enters times
        ``sigmoid(w . x)``, one number a token, ``w`` stored as ``[1, hidden]``.
        ``tensor_names`` maps ``router``, ``router_bias``, ``correction``, ``gate``, ``up``, ``down``,
        ``shared`` (a prefix) and ``shared_gate`` to names behind ``prefix``; the experts' names hold ``{e}`` for
        the expert's number."""
        super().__init__(prefix)
        if scores not in ("softmax", "sigmoid"):
            raise ValueError(f"{prefix}: scores {scores!r} is neither 'softmax' nor 'sigmoid'")
        self.scores, self.groups, self.keep_groups, self.group_top = scores, int(groups), int(keep_groups), int(group_top)
        self.weight_scale, self.sum_eps, self.limit = float(weight_scale), float(sum_eps), float(limit)
        self.shared_limit = self.limit if shared_limit is None else float(shared_limit)
        self.has_shared_gate = bool(shared_gate)
        if self.groups < 1 or not 1 <= self.keep_groups <= self.groups or (int(experts) + int(identity)) % self.groups:
            raise ValueError(f"{prefix}: {groups} groups (of which {keep_groups} are kept) do not divide the router's outputs")
        if activation == "swish_clamped" and not gated:
            raise ValueError(f"{prefix}: the clamped activation is a gated one")
        if softmax_over not in ("all", "chosen"):
            raise ValueError(f"{prefix}: softmax_over {softmax_over!r} is neither 'all' nor 'chosen'")
        self.gated, self.has_router_bias, self.over_chosen = bool(gated), bool(router_bias), softmax_over == "chosen"
        self.shared_intermediate = int(shared_intermediate)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.experts, self.top, self.identity = int(experts), int(top), int(identity)
        if self.experts < 0 or self.identity < 0 or not 0 < self.top <= self.experts + self.identity:
            raise ValueError(f"{prefix}: top {top} of {experts} experts and {identity} identity experts")
        if activation not in K.EXPERT_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(K.EXPERT_ACTIVATIONS)}")
        self.activation, self.has_correction, self.renormalise = activation, bool(correction), bool(renormalise)
        names = dict(router="router", router_bias="router.b", correction="correction", gate="e{e}.gate", up="e{e}.up",
                     down="e{e}.down", shared="shared.", shared_gate="shared.sg")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.outputs = self.experts + self.identity
        self.shared = None
        if self.shared_intermediate > 0:
            if activation not in K.GATED_ACTIVATIONS:
                raise ValueError(f"{prefix}: the expert every token uses runs with one of {sorted(K.GATED_ACTIVATIONS)}")
            from .mlp import SwiGLU
            self.shared = SwiGLU(self.names["shared"], hidden_size=self.hidden_size,
                                 intermediate_size=self.shared_intermediate, activation=activation,
                                 limit=self.shared_limit, tensor_names=dict(gate="gate", up="up", down="down"))
        if self.has_shared_gate and self.shared is None:
            raise ValueError(f"{prefix}: a gate without the expert every token uses")

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, I = self.names, self.hidden_size, self.intermediate_size
        specs = {n["router"]: TensorSpec((self.outputs, W))}
        if self.has_correction:
            specs[n["correction"]] = TensorSpec((self.outputs,), init="zeros", role="vector")
        if self.has_router_bias:
            specs[n["router_bias"]] = TensorSpec((self.outputs,), init="zeros", role="vector")
        for e in range(self.experts):
            if self.gated:
                specs[n["gate"].format(e=e)] = TensorSpec((I, W))
            specs[n["up"].format(e=e)] = TensorSpec((I, W))
            specs[n["down"].format(e=e)] = TensorSpec((W, I))
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        if self.has_shared_gate:
            specs[n["shared_gate"]] = TensorSpec((1, W))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        self.router = tensors[n["router"]].contiguous()             # its logits are formed in 32-bit (ops.kernels.small_product_f32)
        self.correction = tensors[n["correction"]].float().contiguous() if self.has_correction else None
        self.router_bias = tensors[n["router_bias"]].float().contiguous() if self.has_router_bias else None
        if self.shared is not None:
            self.shared.load(tensors)
        # the shared expert's gate is one more row of the router's product: one launch makes both in 32-bit
        self.shared_gate = tensors[n["shared_gate"]].contiguous() if self.has_shared_gate else None
        if self.shared_gate is not None:
            self.router = torch.cat([self.router, self.shared_gate.to(self.router.dtype)], dim=0).contiguous()
            if self.router_bias is not None:
                self.router_bias = torch.cat([self.router_bias, self.router_bias.new_zeros(1)]).contiguous()
        if self.experts and self.gated:
            # rows 2 j and 2 j + 1 of an expert's first matrix: output j's gate row and its up row
            ups = []
            for e in range(self.experts):
                g, u = tensors[n["gate"].format(e=e)], tensors[n["up"].format(e=e)]
                ups.append(torch.stack([g, u], dim=1).reshape(2 * g.shape[0], g.shape[1]))
            self.w_up = torch.stack(ups).contiguous()
            self.w_down = torch.stack([tensors[n["down"].format(e=e)] for e in range(self.experts)]).contiguous()
        elif self.experts:
            self.w_up = torch.stack([tensors[n["up"].format(e=e)] for e in range(self.experts)]).contiguous()
            self.w_down = torch.stack([tensors[n["down"].format(e=e)] for e in range(self.experts)]).contiguous()
        else:
            self.w_up = self.w_down = None

    def activation_elements(self) -> int:
        return self.outputs + self.top * (2 * self.intermediate_size + 2 * self.hidden_size) + self.hidden_size \
            + (self.shared.activation_elements() + self.hidden_size if self.shared is not None else 0)

    def forward(self, x, ctx: MixerContext, tail=None):
        T, dev = x.shape[0], x.device
        cols = self.router.shape[0]              # the router's outputs, and the shared expert's gate behind them
        product = K.small_product_f32(x, self.router, torch.empty((T, cols), dtype=torch.float32, device=dev),
                                      bias=self.router_bias)
        logits = product[:, :self.outputs]
        idx = torch.empty((T, self.top), dtype=torch.int32, device=dev)
        wgt = torch.empty((T, self.top), dtype=torch.float32, device=dev)
        K.moe_route(logits, self.correction, self.top, idx, wgt, self.renormalise, over_chosen=self.over_chosen,
                    scores=self.scores, groups=self.groups, keep_groups=self.keep_groups, group_top=self.group_top,
                    weight_scale=self.weight_scale, sum_eps=self.sum_eps)
        if RoutedExperts.on_route is not None and not torch.cuda.is_current_stream_capturing():
            RoutedExperts.on_route(self, idx)
        slots = T * self.top
        rows = torch.empty((slots, self.hidden_size), dtype=torch.float32, device=dev)
        if self.experts:
            tiles = K.moe_tiles(slots, self.experts)
            sorted_slot = torch.empty(tiles * K.MOE_TILE, dtype=torch.int32, device=dev)
            tile_expert = torch.empty(tiles, dtype=torch.int32, device=dev)
            K.moe_align(idx, self.experts, sorted_slot, tile_expert)
            act = torch.empty((tiles * K.MOE_TILE, self.intermediate_size), dtype=x.dtype, device=dev)
            K.moe_expert_rows(x, self.w_up, act, sorted_slot, tile_expert, self.top, activation=self.activation,
                              gated=self.gated, limit=self.limit)
            K.moe_expert_rows(act, self.w_down, rows, sorted_slot, tile_expert, self.top, slot_weight=wgt)
        out = torch.empty_like(x)
        extra = self.shared.forward(x, ctx) if self.shared is not None else None
        # one number a token, in 32-bit; its sigmoid is taken where the rows are added
        gate = product[:, self.outputs] if self.shared_gate is not None else None
        return K.moe_combine(x, rows, idx, wgt, self.experts, out, extra=extra, extra_gate=gate)
