"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` (reference: ``base/src/kernels.cu:10-36``).

The weight multiplies as stored (no ``1 + w``).  ``forward`` can fuse the residual add that
comes before the norm (``delta``) and a gather of rows (``row_idx``).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import NORMS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import Norm, PendingMix


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    takes_partial_sums = True       # ``delta`` may be ops.kernels.PartialSums (bf16 streams)

    def __init__(self, prefix: str, *, width: int, eps: float, weight_name: str = "weight"):
        super().__init__(prefix)
        self.width, self.eps = int(width), float(eps)
        self.weight_name = prefix + weight_name
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.weight_name: TensorSpec((self.width,), init="norm", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name].contiguous()

    def prepared_by_product(self):
        return (self.weight, self.width, self.eps)

    def activation_elements(self) -> int:
        return self.width

    def into_stream(self, stream, y, copy=None) -> None:
        K.norm_into_stream(stream, y, self.weight, self.eps, copy)

    def forward(self, x, out=None, delta=None, row_idx=None):
        if out is None:
            rows = x.shape[0] if row_idx is None else row_idx.shape[0]
            out = torch.empty((rows, self.width), dtype=x.dtype, device=x.device)
        if isinstance(delta, K.PartialSums) and (x.dtype != torch.bfloat16 or self.width % 8):
            delta = delta.materialize()
        return K.rmsnorm(x, self.weight, self.eps, out, delta=delta, row_idx=row_idx)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """``y = (x - mean) / sqrt(var + eps) * w`` with the variance as the mean of the squared
    deviations; a weight and, optionally, a bias.  Statistics are fp32.  The rows it reads may be an fp32 stream
    while it writes ``out_dtype`` rows (the type the products behind it take).  ``delta`` may be one
    branch output or a tuple of two: they are added to ``x`` in place first.  ``forward_pair``
    writes two normalised copies, this norm's and a ``twin``'s (same width and eps, another
    weight), from one pass and one set of statistics."""

    graph_safe = True

    def __init__(self, prefix: str, *, width: int, eps: float, weight_name: str = "weight",
                 out_dtype: Optional[str] = None, center: bool = True, weight_offset: float = 0.0,
                 bias_name: Optional[str] = None, streams: int = 1):
        """``center=False``: the mean is not taken off (``x / sqrt(mean(x^2) + eps) * w``, an RMS norm
        over a stream of another type than the products').  ``weight_offset``: the weight is stored
        around zero and multiplies as ``weight_offset + w`` (the sum is formed once, in 32-bit).
        ``bias_name``: the norm has a bias, ``... * w + b``.  ``streams``: the rows it reads hold so
        many copies of the stream side by side (32-bit), and what is normed is their sum; a pending
        :class:`~.base.PendingMix` enters the copies first.  A norm with a bias or over several copies
        reads a 32-bit stream (``ops.kernels.hyper_step``)."""
        super().__init__(prefix)
        self.width, self.eps = int(width), float(eps)
        self.weight_name = prefix + weight_name
        self.bias_name = None if bias_name is None else prefix + bias_name
        self.streams = int(streams)
        if (self.bias_name is not None or self.streams > 1) and (not center or weight_offset):
            raise ValueError(f"{prefix}: a bias or several copies of the stream go with the plain centred form")
        self.bias: Optional[torch.Tensor] = None
        self._ones: Optional[torch.Tensor] = None
        self.out_dtype = {None: None, "bfloat16": torch.bfloat16, "float32": torch.float32}[out_dtype]
        self.center, self.weight_offset = bool(center), float(weight_offset)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {self.weight_name: TensorSpec((self.width,), init="zeros" if self.weight_offset else "norm", role="vector")}
        if self.bias_name is not None:
            specs[self.bias_name] = TensorSpec((self.width,), init="normal", role="vector")
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name].contiguous()
        if self.bias_name is not None:
            self.bias = tensors[self.bias_name].contiguous()
        self._ones = torch.ones(self.streams, dtype=torch.float32, device=self.weight.device)
        if self.weight_offset:
            if self.out_dtype is None:
                self.out_dtype = self.weight.dtype          # the products behind the norm take the stored type
            self.weight = (self.weight.float() + self.weight_offset).contiguous()

    def activation_elements(self) -> int:
        return self.width

    @staticmethod
    def _deltas(delta):
        if delta is None:
            return ()
        return tuple(delta) if isinstance(delta, (tuple, list)) else (delta,)

    @staticmethod
    def _scale(delta) -> float:
        return float(getattr(delta, "scale", 1.0))

    def _out(self, x, row_idx):
        rows = x.shape[0] if row_idx is None else row_idx.shape[0]
        # the products behind a norm take the weights' type; a 32-bit stream of a bf16 model is normalised into bf16
        return torch.empty((rows, self.width), dtype=self.out_dtype or self.weight.dtype, device=x.device)

    def forward(self, x, out=None, delta=None, row_idx=None):
        out = self._out(x, row_idx) if out is None else out
        if self.bias is not None or self.streams > 1 or isinstance(delta, PendingMix):
            if delta is not None and not isinstance(delta, PendingMix):
                raise TypeError(f"{self.prefix}: this norm takes a pending output with its way into the stream's copies")
            if delta is not None and delta.streams != self.streams:
                raise ValueError(f"{self.prefix}: the pending output belongs to a stream of {delta.streams} copies")
            enter = {} if delta is None else dict(y=delta.y, mix=delta.mix, out_w=delta.out_w, mult=delta.mult)
            return K.hyper_step(x, self.streams, in_w=self._ones, norm_weight=self.weight, norm_bias=self.bias,
                                eps=self.eps, out=out, row_idx=row_idx, **enter)
        return K.layernorm(x, self.weight, self.eps, out, deltas=self._deltas(delta), row_idx=row_idx,
                           rms=not self.center, delta_scale=self._scale(delta))

    def into_stream(self, stream, y, copy=None) -> None:
        if self.center:
            raise NotImplementedError("only the form without the mean taken off norms a branch output into the stream")
        K.norm_into_stream(stream, y, self.weight, self.eps, copy)

    def forward_pair(self, twin: "LayerNorm", x, delta=None):
        if twin.width != self.width or twin.eps != self.eps or twin.weight.dtype != self.weight.dtype \
                or twin.center != self.center:
            raise ValueError("two norms share a pass only with the same form, width, eps and weight type")
        out, out2 = self._out(x, None), self._out(x, None)
        K.layernorm(x, self.weight, self.eps, out, deltas=self._deltas(delta), weight2=twin.weight, out2=out2,
                    rms=not self.center, delta_scale=self._scale(delta))
        return out, out2
