"""Grouped-query causal attention over the paged cache (the Llama mixer).

Per token (reference order, ``base/src/engine.cu:652-762``): Q, K, V projections without bias
-> position encoding of Q and K -> K and V written to the cache -> scores ``q.k * scale`` over
the request's keys up to the token's own position (optionally only the last ``window``),
softmax in fp32 -> ``P V`` -> output projection.  ``kv_head = q_head // (num_heads / num_kv_heads)``.

The three projection matrices are joined at load time into one ``[nq*d + 2*nkv*d, hidden]``
matrix, so the step runs one product instead of three.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..models.spec import PartSpec, TensorSpec
from ..ops import attention as attn_ops
from ..ops import kernels as K
from ..ops.gemm_bf16 import SKINNY_MAX_ROWS
from .base import (BranchTail, KVCacheSpec, Mixer, MixerContext, NormedRows, ProjectedMixer,
                   attention_cache_spec)
from .linear import Linear


class EncodedQKV:
    """The joined Q/K/V projection with position encoding and cache write: what every mixer that
    attends over cached keys does first.  It owns the choice between one product that does all of
    it in its epilogue (few rows, an encoding that is a rotate-half rotation over the whole head,
    or none) and the product followed by the encoding's own kernel, so that a mixer - this one or
    another attention variant - only says ``qkv(x, batch, kv)``."""

    # Above 16 decoded tokens the library's product followed by the attention kernel that rotates and
    # caches inside is ahead of the few-rows product with that work in its epilogue, except for large
    # matrices at many rows.  Whole decode steps at 768 keys, ms, epilogue -> attention kernel:
    # 1B sizes (3,072 x 2,048) 17 / 24 / 32 requests 1.188 / 1.243 / 1.292 -> 1.133 / 1.194 / 1.245;
    # 8 layers of the 3B sizes (5,120 x 3,072) 17 / 32 / 48: 0.855 / 0.929 / 1.040 -> 0.838 / 0.927 / 1.007;
    # 8 layers of the 8B sizes (6,144 x 4,096) 17 / 24: 1.262 / 1.298 -> 1.259 / 1.281, but 32 / 40 / 48:
    # 1.288 / 1.386 / 1.374 -> 1.292 / 1.400 / 1.416.
    ROTATE_LATER_ROWS = 24
    ROTATE_LATER_ELEMENTS = 1 << 24

    def __init__(self, linear: Linear, position, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, value_dim: Optional[int] = None, rotate_later: bool = True):
        self.linear, self.position = linear, position
        # False: the attention call that follows has options the kernel that rotates inside lacks
        self.rotate_later = bool(rotate_later)
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        # values of another size than the keys: only the encoding's own kernel lays such rows out
        self.value_dim = int(head_dim if value_dim is None else value_dim)
        self.pending_rotation = None          # set by a call that left encoding and cache write to the attention kernel

    def __call__(self, x, batch, kv):
        """``x`` [T, hidden] (plain or NormedRows).  Returns a tensor whose first ``nq * d`` columns
        are the position-encoded queries; K (encoded) and V of the step's tokens are in the cache
        when ``kv`` allows writing.  Or, with ``self.pending_rotation`` set to the (cos, sin) tables
        (or (None, None)), the joined projection as the product left it: encoding and cache write
        are then the attention kernel's (``ops.attention.paged_attention(..., rope=...)``)."""
        self.pending_rotation = None
        tables, rows = None, x.shape[0]
        kernel = self.linear.fused_kernel(rows, x.dtype, rotated=True)
        if self.value_dim != self.head_dim:
            qkv = self.linear(x)
            self.position.apply_and_cache(qkv, batch.positions, self.num_heads, self.num_kv_heads,
                                          self.head_dim, kv, value_dim=self.value_dim)
            return qkv
        if kernel == Linear.GEMV and not K.gemv_qkv_rope_supported(rows, self.hidden_size, self.head_dim):
            kernel = Linear.FEW_ROWS if self.linear.tiled is not None else None
        if kernel == Linear.FEW_ROWS and not K.gemm_skinny_qkv_rope_supported(rows, self.hidden_size, self.head_dim):
            kernel = None
        if (kernel == Linear.FEW_ROWS and rows > SKINNY_MAX_ROWS
                and (rows <= self.ROTATE_LATER_ROWS or self.linear.weight.numel() <= self.ROTATE_LATER_ELEMENTS)
                and self.rotate_later and attn_ops.rotates_in_kernel(batch, kv, self.num_heads, self.num_kv_heads, self.head_dim, x.dtype)):
            kernel = None
        if kernel is not None:
            tables = self.position.rotate_half_tables(x.device, self.head_dim)
        if tables is None:
            qkv = self.linear(x)
            # decoded tokens only: rotation and cache write go into the attention kernel, which
            # takes the product as it is (one launch less per layer where the product is the library's)
            later = self.position.rotate_half_tables(x.device, self.head_dim)
            if later is not None and self.rotate_later and attn_ops.rotates_in_kernel(batch, kv, self.num_heads, self.num_kv_heads,
                                                                self.head_dim, qkv.dtype):
                self.pending_rotation = later
                return qkv
            self.position.apply_and_cache(qkv, batch.positions, self.num_heads, self.num_kv_heads,
                                          self.head_dim, kv)
            return qkv
        write = kv is not None and kv.writes
        q = torch.empty((rows, self.num_heads * self.head_dim), dtype=torch.bfloat16, device=x.device)
        norm = {}
        if isinstance(x, NormedRows):
            norm = dict(sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
            x = x.scaled
        product, weight = ((K.gemv_qkv_rope, self.linear.weight) if kernel == Linear.GEMV
                           else (K.gemm_skinny_qkv_rope, self.linear.tiled))
        product(x, weight, q, self.num_heads, self.num_kv_heads, self.head_dim,
                batch.positions, tables[0], tables[1],
                kv.k_cache if write else None, kv.v_cache if write else None,
                kv.slot_mapping if write else None, kv.page_size if kv is not None else 0, **norm)
        return q


@MIXERS.register("gqa_attention")
class GQAAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, position: PartSpec, window: int = 0, keep_first: int = 0,
                 value_dim: Optional[int] = None, tensor_names: Optional[Dict[str, str]] = None):
        """``window`` > 0: a query at position i sees key j only when ``i - j < window`` or
        ``j < keep_first`` (the first positions of a request stay visible, at their true places).
        ``value_dim``: the size of a value head where it is not ``head_dim``.  ``tensor_names``
        maps ``q``, ``k``, ``v``, ``o`` to the names (behind ``prefix``) of the four matrices."""
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads is not a multiple of {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.scale, self.window = head_dim, float(scale), int(window)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        self.value_dim = int(head_dim if value_dim is None else value_dim)
        names = dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", o="o_proj.weight")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.position = POSITION_ENCODINGS.get(position.kind)(**position.params)
        self.qkv: Optional[EncodedQKV] = None
        self.o: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, d, dv = self.names, self.head_dim, self.value_dim
        return {
            n["q"]: TensorSpec((self.num_heads * d, self.hidden_size)),
            n["k"]: TensorSpec((self.num_kv_heads * d, self.hidden_size)),
            n["v"]: TensorSpec((self.num_kv_heads * dv, self.hidden_size)),
            n["o"]: TensorSpec((self.hidden_size, self.num_heads * dv)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        q, k, v = (tensors[self.names[n]] for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError(f"{self.prefix}: q/k/v projection weights are stored in different dtypes")
        self.qkv = EncodedQKV(Linear(torch.cat([q, k, v], dim=0)), self.position, self.hidden_size,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                              rotate_later=self.keep_first == 0)
        self.o = Linear(tensors[self.names["o"]])

    def kv_cache_spec(self) -> KVCacheSpec:
        return attention_cache_spec(self.num_kv_heads, self.head_dim,
                                    kind="window" if self.window > 0 else "full", window=self.window,
                                    value_dim=self.value_dim, keep_first=self.keep_first)

    fuses_tail = True

    def activation_elements(self) -> int:
        # the joined projection, the attention output and the output projection
        return ((self.num_heads + self.num_kv_heads) * (self.head_dim + self.value_dim)
                + self.hidden_size)

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        """``x`` may be NormedRows (the input norm is then finished inside the QKV product); with
        a ``tail`` the output projection adds into the residual stream and prepares the next
        norm when the shapes allow, and NormedRows are returned instead of the plain output."""
        batch, kv = ctx.batch, ctx.kv
        qkv = self.qkv(x, batch, kv)
        out = torch.empty((x.shape[0], self.num_heads * self.value_dim), dtype=x.dtype, device=x.device)
        # an output projection that adds the key ranges' partial results up itself (one or two
        # decoded tokens) is told so: the attention kernel may then leave them unmerged
        plain = self.keep_first == 0 and self.value_dim == self.head_dim
        max_parts = self.o.takes_attention_partials(x.shape[0], x.dtype, tail, self.head_dim) \
            if self.qkv.pending_rotation is None and plain else 0
        out = attn_ops.paged_attention(qkv, out, kv, batch, self.num_heads, self.num_kv_heads,
                                       self.head_dim, self.scale, self.window, rope=self.qkv.pending_rotation,
                                       max_parts=max_parts, keep_first=self.keep_first, value_dim=self.value_dim)
        if tail is not None:
            fused = self.o.into_residual(out, tail)
            if fused is not None:
                return fused
        return self.o(out)


@MIXERS.register("gated_gqa_attention")
class GatedGQAAttention(ProjectedMixer):
    """Grouped-query causal attention over the paged cache with what :class:`GQAAttention` leaves
    out: biases on the q, k and v projections (added where the heads are rotated and cached) and an
    output gate - the concatenated heads times ``sigmoid(W_g x)``, element by element, before the
    output projection.  The position encoding is a part like everywhere (a rotation of the first
    elements of a head passes the rest unchanged); window, kept first positions and a value size of
    its own are the options :func:`~..ops.attention.paged_attention` has.  As a
    :class:`~.base.ProjectedMixer` it runs alone or beside other mixers on the same input."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, position: PartSpec, value_dim: Optional[int] = None, window: int = 0,
                 keep_first: int = 0, bias: bool = False, gate: Optional[str] = "sigmoid",
                 qk_norm: Optional[str] = None, norm_eps: float = 0.0, sink: bool = False,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``bias``: q, k and v have biases named like their matrices with ``bias_suffix`` added.
        ``gate``: ``"sigmoid"``, ``"silu"`` or ``None``.  ``qk_norm``: every query and key head passes an
        RMS norm (``x / sqrt(mean(x^2) + norm_eps) * w`` with a weight of ``head_dim`` elements for the
        queries and one for the keys, shared by the heads) ``"before_rotation"`` or ``"after_rotation"``;
        the keys lie in the cache normed and rotated.  ``sink``: a stored number per query head whose
        exponential is one more term of every softmax denominator (it has no key and no value and is
        not scaled).  ``tensor_names`` maps ``q k v g o q_norm k_norm sink`` and ``bias_suffix`` to names
        behind ``prefix``."""
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads is not a multiple of {num_kv_heads} kv heads")
        if gate not in (None, "sigmoid", "silu"):
            raise ValueError(f"output gate {gate!r} is not one of None, 'sigmoid', 'silu'")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.scale, self.window = int(head_dim), float(scale), int(window)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        self.value_dim = int(head_dim if value_dim is None else value_dim)
        self.bias, self.gate = bool(bias), gate
        if qk_norm not in (None, "before_rotation", "after_rotation"):
            raise ValueError(f"qk_norm {qk_norm!r} is not one of None, 'before_rotation', 'after_rotation'")
        self.qk_norm, self.norm_eps, self.sink = qk_norm, float(norm_eps), bool(sink)
        self.q_weight = self.k_weight = self.sinks = None
        names = dict(q="q", k="k", v="v", g="g", o="o", bias_suffix=".b", q_norm="q.norm", k_norm="k.norm", sink="sink")
        names.update(tensor_names or {})
        self.bias_suffix = names.pop("bias_suffix")
        self.names = {key: prefix + name for key, name in names.items()}
        self.position = POSITION_ENCODINGS.get(position.kind)(**position.params)
        self.inner_width = self.num_heads * self.value_dim
        self.qkv_width = (self.num_heads + self.num_kv_heads) * self.head_dim + self.num_kv_heads * self.value_dim

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, d, dv, W = self.names, self.head_dim, self.value_dim, self.hidden_size
        specs = {n["q"]: TensorSpec((self.num_heads * d, W)), n["k"]: TensorSpec((self.num_kv_heads * d, W)),
                 n["v"]: TensorSpec((self.num_kv_heads * dv, W)), n["o"]: TensorSpec((W, self.inner_width))}
        if self.gate is not None:
            specs[n["g"]] = TensorSpec((self.inner_width, W))
        if self.bias:
            for key in "qkv":
                specs[n[key] + self.bias_suffix] = TensorSpec((specs[n[key]].shape[0],), init="normal", role="vector")
        if self.qk_norm is not None:
            specs[n["q_norm"]] = TensorSpec((d,), init="norm", role="vector")
            specs[n["k_norm"]] = TensorSpec((d,), init="norm", role="vector")
        if self.sink:
            specs[n["sink"]] = TensorSpec((self.num_heads,), init="normal", role="vector")
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        if self.qk_norm is not None:        # norms and the softmax's terms are 32-bit
            self.q_weight, self.k_weight = tensors[n["q_norm"]].float().contiguous(), tensors[n["k_norm"]].float().contiguous()
        if self.sink:
            self.sinks = tensors[n["sink"]].float().contiguous()
        rows = [tensors[n[key]] for key in "qkv"] + ([tensors[n["g"]]] if self.gate is not None else [])
        self._w_in = torch.cat(rows, dim=0).contiguous()
        self._w_out = tensors[n["o"]]
        self.qkv_bias = torch.cat([tensors[n[key] + self.bias_suffix] for key in "qkv"]).contiguous() if self.bias else None
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def kv_cache_spec(self) -> KVCacheSpec:
        return attention_cache_spec(self.num_kv_heads, self.head_dim, kind="window" if self.window > 0 else "full",
                                    window=self.window, value_dim=self.value_dim, keep_first=self.keep_first)

    def activation_elements(self) -> int:
        return self.qkv_width + 3 * self.inner_width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, kv = ctx.batch, ctx.kv
        qkv = y[:, col0:col0 + self.qkv_width]
        write = kv is not None and kv.writes
        cos, sin = self.position.tables(y.device) if hasattr(self.position, "tables") else (None, None)
        K.qk_encode_cache(qkv, batch.positions, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                          cos, sin, getattr(self.position, "pairing", "half") == "interleaved",
                          self.norm_eps if self.qk_norm is not None else getattr(self.position, "unit_norm_eps", None),
                          kv.k_cache if write else None, kv.v_cache if write else None,
                          kv.slot_mapping if write else None, bias=self.qkv_bias, q_weight=self.q_weight,
                          k_weight=self.k_weight, norm_first=self.qk_norm == "before_rotation")
        direct = self.gate is None and mul == 1.0 and out_col0 == 0 and out.shape[1] == self.inner_width
        heads = out if direct else torch.empty((y.shape[0], self.inner_width), dtype=y.dtype, device=y.device)
        attn_ops.paged_attention(qkv, heads, kv, batch, self.num_heads, self.num_kv_heads, self.head_dim, self.scale,
                                 self.window, keep_first=self.keep_first, value_dim=self.value_dim, sinks=self.sinks)
        if not direct:
            if self.gate is None:
                # the heads times the constant, into their columns of the wider buffer
                K.head_norm_gate(heads, None, 0.0, None, 0, out, out_col0, self.num_heads, self.value_dim, None, mul)
            else:
                K.head_norm_gate(heads, None, 0.0, y, col0 + self.qkv_width, out, out_col0, self.num_heads,
                                 self.value_dim, self.gate, mul)


@MIXERS.register("normed_gqa_attention")
class NormedGQAAttention(Mixer):
    """Grouped-query causal attention whose queries and keys pass an RMS norm per head (a weight
    of ``head_dim`` elements for the queries and one for the keys, shared by the heads) before the
    scores are taken: ``q <- q / sqrt(mean(q^2) + eps) * w_q``, likewise k; the keys lie in the cache
    normed.  The position encoding is a part as everywhere (``"none"``: positions do not enter the
    scores); a rotation is applied before the norm.  Masks: all earlier keys, a ``window`` (with kept
    first positions), or ``chunk``: a query sees a key only inside its own run of ``chunk``
    positions counted from the request's position 0 - wherever a prompt was cut into steps.

    ``shared_kv``: the mixer has no key and value tensors; it attends, with queries, norm, mask and
    output matrix of its own, over what another layer call wrote to the cache slot it is given (the
    run order names that slot with ``writes_cache=False``)."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, norm_eps: float, position: Optional[PartSpec] = None, value_dim: Optional[int] = None,
                 window: int = 0, keep_first: int = 0, chunk: int = 0, shared_kv: bool = False,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``q k v o q_norm k_norm`` to names behind ``prefix``."""
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads is not a multiple of {num_kv_heads} kv heads")
        if window > 0 and chunk > 0:
            raise ValueError(f"{prefix}: either a window or chunks")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.scale, self.norm_eps = int(head_dim), float(scale), float(norm_eps)
        self.value_dim = int(head_dim if value_dim is None else value_dim)
        self.window, self.chunk = int(window), int(chunk)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        self.shared_kv = bool(shared_kv)
        names = dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        position = position or PartSpec("none")
        self.position = POSITION_ENCODINGS.get(position.kind)(**position.params)
        self.in_linear: Optional[Linear] = None
        self.o: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, d, dv, W = self.names, self.head_dim, self.value_dim, self.hidden_size
        specs = {n["q"]: TensorSpec((self.num_heads * d, W)), n["o"]: TensorSpec((W, self.num_heads * dv)),
                 n["q_norm"]: TensorSpec((d,), init="norm", role="vector")}
        if not self.shared_kv:
            specs[n["k"]] = TensorSpec((self.num_kv_heads * d, W))
            specs[n["v"]] = TensorSpec((self.num_kv_heads * dv, W))
            specs[n["k_norm"]] = TensorSpec((d,), init="norm", role="vector")
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        rows = [tensors[n["q"]]] if self.shared_kv else [tensors[n[key]] for key in "qkv"]
        if len({r.dtype for r in rows}) != 1:
            raise ValueError(f"{self.prefix}: q/k/v projection weights are stored in different dtypes")
        self.in_linear = Linear(torch.cat(rows, dim=0) if len(rows) > 1 else rows[0])
        self.o = Linear(tensors[n["o"]])
        self.q_weight = tensors[n["q_norm"]].float().contiguous()
        self.k_weight = None if self.shared_kv else tensors[n["k_norm"]].float().contiguous()

    def kv_cache_spec(self) -> KVCacheSpec:
        # (a chunked layer keeps all its pages: a layer that shares the slot may see them with another mask)
        return attention_cache_spec(self.num_kv_heads, self.head_dim, kind="window" if self.window > 0 else "full",
                                    window=self.window, value_dim=self.value_dim, keep_first=self.keep_first)

    def activation_elements(self) -> int:
        return (self.num_heads + self.num_kv_heads) * (self.head_dim + self.value_dim) + self.hidden_size

    def forward(self, x, ctx: MixerContext):
        batch, kv = ctx.batch, ctx.kv
        if kv is None:
            raise K.KernelError(f"{self.prefix}: the mixer has no cache view")
        if self.shared_kv and kv.writes:
            raise K.KernelError(f"{self.prefix}: a layer without keys and values of its own only reads its cache slot")
        y = self.in_linear(x)
        write = kv.writes and not self.shared_kv
        cos, sin = self.position.tables(y.device) if hasattr(self.position, "tables") else (None, None)
        K.qk_encode_cache(y, batch.positions, self.num_heads, 0 if self.shared_kv else self.num_kv_heads, self.head_dim,
                          self.value_dim, cos, sin, getattr(self.position, "pairing", "half") == "interleaved",
                          self.norm_eps, kv.k_cache if write else None, kv.v_cache if write else None,
                          kv.slot_mapping if write else None, q_weight=self.q_weight, k_weight=self.k_weight)
        heads = torch.empty((y.shape[0], self.num_heads * self.value_dim), dtype=y.dtype, device=y.device)
        attn_ops.paged_attention(y, heads, kv, batch, self.num_heads, self.num_kv_heads, self.head_dim, self.scale,
                                 self.window, keep_first=self.keep_first, value_dim=self.value_dim, chunk=self.chunk)
        return self.o(heads)
