"""Mixers run side by side on the same input: ``y = sum_i scale_i * mixer_i(x)``.

Every child is a :class:`~.base.ProjectedMixer`.  All their input projections are joined into one
product over ``x``, every child works on its own columns of the result (attention over the paged
cache, a recurrence over its state, ...) and writes ``scale_i`` times what its output projection
reads into its own columns of one buffer, and all output projections, joined along their inputs,
are one more product: ``sum_i scale_i W_o,i inner_i = [W_o,1 | W_o,2 | ...] [scale_1 inner_1 ;
scale_2 inner_2 ; ...]``.  The cache entry is the one child's that keeps keys and values; the
states of the children lie one behind the other in the call's state row.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..config.registry import MIXERS
from ..models.spec import PartSpec, TensorSpec
from .base import KVCacheSpec, Mixer, MixerContext, ProjectedMixer, StateSpec
from .linear import Linear


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    COLUMN_ALIGN = 8        # kernels that read a child's columns with wide loads need its rows aligned

    def __init__(self, prefix: str = "", *, hidden_size: int, children: Sequence[PartSpec], scales: Sequence[float]):
        super().__init__(prefix)
        self.hidden_size = int(hidden_size)
        if not children or len(children) != len(scales):
            raise ValueError("mixers side by side: one scale per child, at least one child")
        self.children = [MIXERS.get(c.kind)(**c.params) for c in children]
        self.scales = [float(s) for s in scales]
        for c in self.children:
            if not isinstance(c, ProjectedMixer) or c.hidden_size != self.hidden_size:
                raise ValueError(f"{type(c).__name__} cannot stand side by side: it is no projected mixer of width "
                                 f"{self.hidden_size}")
        if sum(c.kv_cache_spec() is not None for c in self.children) > 1:
            raise ValueError("mixers side by side: at most one child may keep keys and values")
        self.inner_width = sum(c.inner_width for c in self.children)
        # a position encoding's tables are limited and checked through the mixer that owns them
        self.position = next((c.position for c in self.children if getattr(c, "position", None) is not None), None)
        self.portion_multiple = 1
        for c in self.children:
            self.portion_multiple = max(self.portion_multiple, int(getattr(c, "portion_multiple", 1)))
        self.w_in: Optional[Linear] = None
        self.w_out: Optional[Linear] = None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(c, "graph_safe", False) for c in self.children)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for c in self.children:
            out.update(c.tensor_specs())
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        ins, outs = [], []
        for c in self.children:
            c.load(tensors)
            w = c.input_weight()
            pad = -w.shape[0] % self.COLUMN_ALIGN
            if pad:         # every child's columns start at a multiple of 16 (or 32) bytes of a row
                w = torch.cat([w, w.new_zeros((pad, w.shape[1]))], dim=0)
            ins.append(w)
            outs.append(c.output_weight())
        if len({w.dtype for w in ins + outs}) != 1:
            raise ValueError(f"{self.prefix}: the children's projection weights are stored in different dtypes")
        self.col0, self.out_col0, self.state_off = [], [], []
        col = ocol = soff = 0
        for c, w in zip(self.children, ins):
            self.col0.append(col)
            self.out_col0.append(ocol)
            self.state_off.append(soff)
            col, ocol, soff = col + w.shape[0], ocol + c.inner_width, soff + c.state_elements()
        self.w_in = Linear(torch.cat(ins, dim=0))
        self.w_out = Linear(torch.cat(outs, dim=1))
        for c in self.children:           # the joined products replace the children's own
            c._in = c._out = None

    def kv_cache_spec(self) -> Optional[KVCacheSpec]:
        return next((s for s in (c.kv_cache_spec() for c in self.children) if s is not None), None)

    def state_spec(self) -> Optional[StateSpec]:
        n = sum(c.state_elements() for c in self.children)
        return StateSpec((n,), torch.float32) if n else None

    def activation_elements(self) -> int:
        return sum(c.activation_elements() for c in self.children)

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        y = self.w_in(x)
        ctx.x = x
        inner = torch.empty((x.shape[0], self.inner_width), dtype=x.dtype, device=x.device)
        for c, col0, out0, soff, scale in zip(self.children, self.col0, self.out_col0, self.state_off, self.scales):
            c.forward_inner(y, col0, ctx, soff, inner, out0, scale)
        return self.w_out(inner)
