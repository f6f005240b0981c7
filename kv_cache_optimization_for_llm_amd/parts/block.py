"""Pre-norm residual block: ``h += mixer(norm1(h)); h += ffn(norm2(h))``
(reference: ``base/src/engine.cu:639-859``).

The sums are made in fp32 and rounded to the storage type.  A branch output is handed on as
``delta`` and added inside the next norm kernel, which sees exactly the rounded sum a separate
residual kernel would have produced.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import BLOCKS, LAYER_INPUTS
from ..models.spec import PartSpec
from ..ops import kernels as K
from ..models.spec import TensorSpec
from .base import Block, BranchTail, MixerContext, Norm, NormedRows, Part, PendingMix, PendingSum, StreamCopy


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


class HyperConnection(Part):
    """How one branch reads and re-enters a residual stream of ``streams`` copies: input weights ``in`` [S]
    (the branch reads ``sum_s in[s] x_s``), a mixing matrix ``mix`` [S, S] indexed [from, to] and output
    weights ``out`` [S] (``x_t <- sum_s mix[s, t] x_s + mult * out[t] * y``).  ``learned=False``: no tensors,
    all of them 1 - with one copy that is the plain residual sum."""

    graph_safe = True

    def __init__(self, prefix: str, *, streams: int, learned: bool = True):
        super().__init__(prefix)
        self.streams, self.learned = int(streams), bool(learned)
        if not self.learned and self.streams != 1:
            raise ValueError(f"{prefix}: several copies of the stream need stored weights")
        self.in_w = self.out_w = self.mix = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if not self.learned:
            return {}
        S, p = self.streams, self.prefix
        return {p + "in": TensorSpec((S,), init="norm", role="vector"),
                p + "out": TensorSpec((S,), init="norm", role="vector"),
                p + "mix": TensorSpec((S, S), init="eye", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor], device=None) -> None:
        if self.learned:
            p = self.prefix
            # the stream and every sum into it are 32-bit: so are these
            self.in_w, self.out_w = tensors[p + "in"].float().contiguous(), tensors[p + "out"].float().contiguous()
            self.mix = tensors[p + "mix"].float().contiguous()
        else:
            self.in_w = self.out_w = torch.ones(1, dtype=torch.float32, device=device)
            self.mix = torch.ones((1, 1), dtype=torch.float32, device=device)


@BLOCKS.register("hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm branches over a residual stream kept in 32-bit as ``streams`` copies of every row, side by side
    (``hidden`` is ``[T, streams * width]``): for the mixer and then the feed-forward, ``u = sum_s in[s] x_s``,
    ``y = branch(norm(u))``, and all copies at once from the old ones ``x_t <- sum_s mix[s, t] x_s + residual_mult
    * out[t] * y``.  The layer's norms are layer norms (weight and, if they have one, bias) whose arithmetic
    runs inside the same pass: one launch (``ops.kernels.hyper_step``) lets the previous branch's output into
    the copies, reads them out and norms - so a layer is two such launches, and the last output travels on as
    :class:`~.base.PendingMix` to whoever reads the stream next.  ``learned=False`` (one copy, no tensors):
    ``x <- x + residual_mult * branch(norm(x))``.  A layer without a feed-forward names only the ``"mixer"``
    norm.  ``connection_names``: the two connections' tensor prefixes behind ``prefix``."""

    graph_safe = True
    NORM_NAMES = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms, *, prefix: str = "", streams: int = 1, learned: bool = True,
                 residual_mult: float = 1.0, connection_names=("hc1.", "hc2.")):
        self.has_ffn = not getattr(feed_forward, "absent", False)
        if not self.has_ffn:
            self.NORM_NAMES = ("mixer",)
        super().__init__(mixer, feed_forward, norms)
        self.streams, self.residual_mult = int(streams), float(residual_mult)
        self.connections = [HyperConnection(prefix + name, streams=streams, learned=learned)
                            for name in connection_names[:2 if self.has_ffn else 1]]
        for norm in self.norms.values():
            if not getattr(norm, "center", False) or getattr(norm, "weight_offset", 0.0):
                raise ValueError("this arrangement runs centred layer norms (weight, optional bias) inside its own pass")

    def parts(self):
        return (*super().parts(), *self.connections)

    def first_norm(self) -> Optional[Norm]:
        return None

    def _read(self, hidden, pending, connection, norm):
        """Lets ``pending`` into the copies, then the branch's input: the normed read-out."""
        if connection.in_w is None or connection.in_w.device != hidden.device:
            connection.load({}, hidden.device)
        x = torch.empty((hidden.shape[0], norm.width), dtype=norm.out_dtype or norm.weight.dtype, device=hidden.device)
        enter = {} if pending is None else dict(y=pending.y, mix=pending.mix, out_w=pending.out_w, mult=pending.mult)
        return K.hyper_step(hidden, self.streams, in_w=connection.in_w, norm_weight=norm.weight, norm_bias=norm.bias,
                            eps=norm.eps, out=x, **enter)

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        if delta is not None and not isinstance(delta, PendingMix):
            raise TypeError("this arrangement takes the stream's copies and a pending output with its way into them")
        if hidden.dtype != torch.float32 or hidden.shape[1] != self.streams * self.norms["mixer"].width:
            raise TypeError(f"the stream must be 32-bit rows of {self.streams} copies")
        first = self.connections[0]
        a = self.mixer.forward(self._read(hidden, delta, first, self.norms["mixer"]), ctx)
        pending = PendingMix(a, first.mix, first.out_w, self.residual_mult, self.streams)
        if self.has_ffn:
            second = self.connections[1]
            f = self.feed_forward.forward(self._read(hidden, pending, second, self.norms["feed_forward"]), ctx)
            pending = PendingMix(f, second.mix, second.out_w, self.residual_mult, self.streams)
        return hidden, pending
