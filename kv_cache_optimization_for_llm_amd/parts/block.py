"""Pre-norm residual block: ``h += mixer(norm1(h)); h += ffn(norm2(h))``
(reference: ``base/src/engine.cu:639-859``).

The sums are made in fp32 and rounded to the storage type.  A branch output is handed on as
``delta`` and added inside the next norm kernel, which sees exactly the rounded sum a separate
residual kernel would have produced.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import BLOCKS, LAYER_INPUTS
from ..models.spec import PartSpec
from ..ops import kernels as K
from .base import Block, BranchTail, MixerContext, Norm, NormedRows, PendingSum, StreamCopy


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    graph_safe = True
    NORM_NAMES = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms):
        super().__init__(mixer, feed_forward, norms)
        self.mixer_norm, self.ffn_norm = self.norms["mixer"], self.norms["feed_forward"]

    def first_norm(self) -> Norm:
        return self.mixer_norm

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        # first norm: already prepared by the previous product, or add-and-normalise here
        if isinstance(delta, NormedRows):
            x = delta if getattr(self.mixer, "fuses_tail", False) else delta.materialize()
        else:
            x = self.mixer_norm.forward(hidden, delta=delta)
        if getattr(self.mixer, "fuses_tail", False):
            a = self.mixer.forward(x, ctx, tail=BranchTail(hidden, self.ffn_norm))
        else:
            a = self.mixer.forward(x, ctx)
        if isinstance(a, NormedRows):               # hidden has taken the mixer's output already
            x = a if getattr(self.feed_forward, "fuses_tail", False) else a.materialize()
        else:
            x = self.ffn_norm.forward(hidden, delta=a)
        if getattr(self.feed_forward, "fuses_tail", False):
            f = self.feed_forward.forward(x, ctx, tail=BranchTail(hidden, next_norm))
        else:
            f = self.feed_forward.forward(x, ctx)
        return hidden, f


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """Both branches read the same stream: ``h += mixer(norm_m(h)) + ffn(norm_f(h))``.

    The two branch outputs are handed on as ``delta`` (a tuple) and added by whatever reads the
    stream next - this block's own norm pass, the next block's, the final norm or an operation
    between layers - in one pass over the stream, in the stream's own type (an fp32 stream stays
    fp32 whatever the branches compute in).  When both norms are of one form with the same width
    and eps (``forward_pair``), one pass writes both normalised copies.  A layer without a
    feed-forward (``"none"``) names only the ``"mixer"`` norm.

    ``shared_norm``: the layer has one norm (``"mixer"``) and both branches read its output.
    ``residual_mult`` m: the branches enter the stream as ``h += m (mixer + ffn)`` - the sum is
    handed on as a :class:`PendingSum` and the reader of the stream multiplies while it adds."""

    graph_safe = True
    NORM_NAMES = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms, *, shared_norm: bool = False, residual_mult: float = 1.0):
        self.has_ffn = not getattr(feed_forward, "absent", False)
        self.shared_norm, self.residual_mult = bool(shared_norm), float(residual_mult)
        if not self.has_ffn or self.shared_norm:
            self.NORM_NAMES = ("mixer",)
        super().__init__(mixer, feed_forward, norms)
        self.mixer_norm = self.norms["mixer"]
        self.ffn_norm = self.norms.get("feed_forward")

    def first_norm(self) -> Optional[Norm]:
        return None             # the stream is handed over as it is, with its pending branch outputs

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        if isinstance(delta, NormedRows):
            raise TypeError("a parallel block takes the stream and plain branch outputs, not prepared rows")
        pair = getattr(self.mixer_norm, "forward_pair", None)
        if self.shared_norm or not self.has_ffn:
            xm = xf = self.mixer_norm.forward(hidden, delta=delta)
        elif pair is not None and type(self.ffn_norm) is type(self.mixer_norm) \
                and (self.ffn_norm.width, self.ffn_norm.eps) == (self.mixer_norm.width, self.mixer_norm.eps):
            xm, xf = pair(self.ffn_norm, hidden, delta=delta)
        else:
            xm = self.mixer_norm.forward(hidden, delta=delta)        # adds the pending outputs to the stream
            xf = self.ffn_norm.forward(hidden)
        a = self.mixer.forward(xm, ctx)
        out = (a, self.feed_forward.forward(xf, ctx)) if self.has_ffn else (a,)
        if self.residual_mult != 1.0:
            return hidden, PendingSum(out, self.residual_mult)
        return hidden, out if self.has_ffn else a


@BLOCKS.register("post_norm")
class PostNormBlock(Block):
    """The norm stands on every branch's OUTPUT: ``h += norm_m(mixer(h)); h += norm_f(ffn(h))``; the
    branches read the stream itself.  ``layer_input`` (a :class:`~..models.spec.PartSpec` of the
    ``LAYER_INPUTS`` registry) names a third branch that runs last and brings something from outside
    the layer - the token's own row of a table - under a norm of its own: ``h += norm_i(input(h))``.
    A layer without a feed-forward (``"none"``) names only the ``"mixer"`` norm.

    Every sum and every norm is one pass (``ops.kernels.norm_into_stream``): it reads the branch's
    output, norms it, adds it to the stream in the stream's own type, and - where the stream is kept in
    32-bit under bfloat16 products - writes the rounded copy that the next branch reads, which is
    handed on to the next block as :class:`~.base.StreamCopy`."""

    graph_safe = True
    NORM_NAMES = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms, *, layer_input: Optional[PartSpec] = None):
        self.has_ffn = not getattr(feed_forward, "absent", False)
        if not self.has_ffn:
            self.NORM_NAMES = ("mixer",)
        super().__init__(mixer, feed_forward, norms)
        self.layer_input = None
        if layer_input is not None:
            self.layer_input = LAYER_INPUTS.get(layer_input.kind)(**layer_input.params)

    def parts(self):
        return (*super().parts(), *((self.layer_input,) if self.layer_input is not None else ()))

    def first_norm(self) -> Optional[Norm]:
        return None

    def _products_dtype(self) -> torch.dtype:
        return self.norms["mixer"].weight.dtype     # vectors take the engine's compute type, like the matrices

    def _into_stream(self, hidden, y, norm):
        """``hidden += norm(y)``; returns the stream as the next branch reads it."""
        if hidden.dtype == self._products_dtype():
            norm.into_stream(hidden, y)
            return hidden
        copy = torch.empty(hidden.shape, dtype=self._products_dtype(), device=hidden.device)
        norm.into_stream(hidden, y, copy)
        return copy

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        if isinstance(delta, StreamCopy):
            h = delta.rows
        elif delta is not None:
            raise TypeError("this arrangement takes the stream as it is, without pending branch outputs")
        elif hidden.dtype == self._products_dtype():
            h = hidden
        else:
            h = K.cast(hidden, torch.empty(hidden.shape, dtype=self._products_dtype(), device=hidden.device))
        h = self._into_stream(hidden, self.mixer.forward(h, ctx), self.norms["mixer"])
        if self.has_ffn:
            h = self._into_stream(hidden, self.feed_forward.forward(h, ctx), self.norms["feed_forward"])
        if self.layer_input is not None:
            h = self._into_stream(hidden, self.layer_input.forward(h, ctx), self.layer_input)
        return hidden, (StreamCopy(h) if h is not hidden else None)
