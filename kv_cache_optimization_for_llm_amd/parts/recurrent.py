"""Mixers that carry a state of fixed size per request instead of keys and values.

Both are :class:`~.base.ProjectedMixer`: one joined input projection, a recurrence over the
request's tokens in order (``csrc/recurrent.hip``: the state ``S [key channels, value channels]``
of every head is fp32, lives in the seat's state row between steps, and everything that enters
the recurrence - decays, step sizes, unit norms - is formed in fp32 from the projection), a norm
of every head's read-out, a gate, and the output projection.  A prompt may be cut anywhere: the
order of every sum depends on the sizes alone.

* :class:`GatedLinearAttention` (``"gated_linear_attention"``):
  ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` with a decay per key channel
  ``alpha = sigmoid(z)^(1 / tau)``, ``z`` a low-rank projection of the input with a bias.
* :class:`GatedDeltaRule` (``"gated_delta_rule"``): ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
  o = S^T q`` with one decay ``g = exp(-exp(A_log) softplus(a + dt_bias))`` and one step size
  ``beta = sigmoid(b)`` per head, unit-norm q and k, and a short causal convolution with silu on
  q, k and v whose last inputs are part of the state.  ``decay="channel"``: the decay has one value
  per head and key channel (a low-rank projection with a bias per channel and a rate per head) and
  multiplies the rows of ``S`` one by one; ``gate_rank``: the output gate is a low-rank projection.
* :class:`LightningAttention` (``"lightning_attention"``): ``S_t = decay_h S_(t-1) + k_t v_t^T``,
  ``o_t = S_t^T q_t`` with one fixed decay a head, silu on q, k and v, and ONE norm over all heads'
  read-outs together.
* :class:`MatrixMemory` (``"matrix_memory"``): a matrix ``S``, a vector ``n`` and a running maximum ``m``
  per head under exponential input and forget gates: ``m' = max(f + m, i)``, ``S <- e^(f + m - m') S +
  e^(i - m') k v^T``, ``n`` likewise with ``k`` alone, ``o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)``.
* :class:`RealGatedLRU` (``"real_gated_lru"``): per channel ``S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t``
  behind a short causal convolution, with gates made by block-diagonal matrices, times a gelu branch.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import MIXERS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import MixerContext, ProjectedMixer


def _names(defaults: Dict[str, str], given: Optional[Dict[str, str]], prefix: str) -> Dict[str, str]:
    names = dict(defaults)
    names.update(given or {})
    return {key: prefix + name for key, name in names.items()}


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(ProjectedMixer):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, tau: float,
                 norm_eps: float, decay_rank: Optional[int] = None, query_scale: Optional[float] = None,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``decay_rank``: the inner size of the decay's low-rank projection; ``None`` takes it from the
        stored tensors.  ``query_scale``: what q is multiplied by (default ``head_dim^-1/2``).
        ``tensor_names`` maps ``q k v g o norm a1 a2 a2_bias`` to names behind ``prefix``."""
        super().__init__(prefix)
        if tau <= 0:
            raise ValueError(f"{prefix}: tau {tau} must be positive")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.query_scale = float(head_dim) ** -0.5 if query_scale is None else float(query_scale)
        self.inner_width = self.num_heads * self.value_dim
        self.names = _names(dict(q="q", k="k", v="v", g="g", o="o", norm="norm", a1="a1", a2="a2", a2_bias="a2.b"),
                            tensor_names, prefix)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, hd, hv, r = self.names, self.hidden_size, self.num_heads * self.head_dim, self.inner_width, self.decay_rank
        return {
            n["q"]: TensorSpec((hd, W)), n["k"]: TensorSpec((hd, W)), n["v"]: TensorSpec((hv, W)),
            n["g"]: TensorSpec((hv, W)), n["o"]: TensorSpec((W, hv)),
            n["norm"]: TensorSpec((self.value_dim,), init="norm", role="vector"),
            n["a1"]: TensorSpec((r, W)), n["a2"]: TensorSpec((hd, r)),
            n["a2_bias"]: TensorSpec((hd,), init="zeros", role="vector"),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = {key: tensors[name] for key, name in self.names.items()}
        if t["a1"].shape[0] != t["a2"].shape[1]:
            raise ValueError(f"{self.prefix}: the decay's two matrices do not fit each other: "
                             f"{tuple(t['a1'].shape)} and {tuple(t['a2'].shape)}")
        self._w_in = torch.cat([t["q"], t["k"], t["v"], t["g"], t["a1"]], dim=0).contiguous()
        self._w_out = t["o"]
        self.rank = int(t["a1"].shape[0])
        hd, hv = self.num_heads * self.head_dim, self.inner_width
        self.q_off, self.k_off, self.v_off, self.g_off, self.a_off = 0, hd, 2 * hd, 2 * hd + hv, 2 * hd + 2 * hv
        # decays are formed in 32-bit: the second matrix of the low-rank projection multiplies in fp32
        self.a2 = t["a2"].contiguous()
        self.a2_bias = t["a2_bias"].float().contiguous()
        self.norm_weight = t["norm"].float().contiguous()
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def state_elements(self) -> int:
        return self.num_heads * self.head_dim * self.value_dim

    def activation_elements(self) -> int:
        return 3 * self.num_heads * self.head_dim + 5 * self.inner_width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, T = ctx.batch, y.shape[0]
        # the decays: the low-rank projection's second half, its bias, sigmoid and power in one 32-bit pass
        alpha = K.small_product_f32(y[:, col0 + self.a_off:col0 + self.a_off + self.rank], self.a2,
                                    torch.empty((T, self.num_heads * self.head_dim), dtype=torch.float32, device=y.device),
                                    bias=self.a2_bias, decay_tau=self.tau)
        o = torch.empty((T, self.inner_width), dtype=torch.float32, device=y.device)
        K.gated_linear_attention(y, col0 + self.q_off, col0 + self.k_off, col0 + self.v_off, alpha, self.query_scale, o,
                                 ctx.state, state_off, batch.entry_q_start, batch.entry_seat, self.num_heads,
                                 self.head_dim, self.value_dim)
        K.head_norm_gate(o, self.norm_weight, self.norm_eps, y, col0 + self.g_off, out, out_col0, self.num_heads,
                         self.value_dim, "silu", mul)


@MIXERS.register("gated_delta_rule")
class GatedDeltaRule(ProjectedMixer):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int, conv_taps: int, norm_eps: float, unit_eps: float = 1e-6,
                 decay: str = "head", decay_rank: Optional[int] = None, gate: str = "silu",
                 gate_rank: Optional[int] = None, low_rank_gate: bool = False,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``num_kv_heads`` query/key heads serve ``num_heads`` value heads (head h uses q/k head
        ``h // (num_heads / num_kv_heads)``).  ``conv_taps``: length of the causal convolution on q, k, v
        (1: none but the silu).  ``decay``: ``"head"`` - one decay a head, ``exp(-exp(A_log_h) softplus(W_a x +
        dt_bias_h))`` - or ``"channel"`` - one per head and key channel, ``exp(-exp(A_log_h) softplus(W_a2 (W_a1
        x) + dt_bias))`` with ``dt_bias`` of ``heads * head_dim`` values and the second product in 32-bit
        (``decay_rank``: the inner size, ``None`` takes it from the stored tensors).  ``gate``: the activation
        of the output gate (``"silu"`` or ``"sigmoid"``); ``low_rank_gate``: the gate is ``W_g2 (W_g1 x)``
        (``gate_rank`` its inner size, ``None`` from the stored tensors).  ``tensor_names`` maps ``q k v q_conv
        k_conv v_conv beta decay A_log dt_bias g norm o`` - and ``a1 a2 g1 g2`` - to names behind ``prefix``."""
        super().__init__(prefix)
        if decay not in ("head", "channel"):
            raise ValueError(f"{prefix}: decay {decay!r} is neither 'head' nor 'channel'")
        if gate not in K.HEAD_GATES:
            raise ValueError(f"{prefix}: gate {gate!r} is not one of {sorted(K.HEAD_GATES)}")
        self.channel_decay, self.gate, self.low_rank_gate = decay == "channel", gate, bool(low_rank_gate)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.gate_rank = None if gate_rank is None else int(gate_rank)
        if num_heads % num_kv_heads:
            raise ValueError(f"{prefix}: {num_heads} heads is not a multiple of {num_kv_heads} key heads")
        if not 1 <= conv_taps <= 17:
            raise ValueError(f"{prefix}: a convolution of {conv_taps} taps (1..17 are built)")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.conv_taps = int(head_dim), int(value_dim), int(conv_taps)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.inner_width = self.num_heads * self.value_dim
        self.conv_channels = 2 * self.num_kv_heads * self.head_dim + self.inner_width
        self.names = _names(dict(q="q", k="k", v="v", q_conv="q.conv", k_conv="k.conv", v_conv="v.conv", beta="b",
                                 decay="a", A_log="A_log", dt_bias="dt_bias", g="g", norm="norm", o="o",
                                 a1="a1", a2="a2", g1="g1", g2="g2"),
                            tensor_names, prefix)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, gd, hv, H, taps = self.names, self.hidden_size, self.num_kv_heads * self.head_dim, self.inner_width, \
            self.num_heads, self.conv_taps
        specs = {
            n["q"]: TensorSpec((gd, W)), n["k"]: TensorSpec((gd, W)), n["v"]: TensorSpec((hv, W)),
            n["q_conv"]: TensorSpec((gd, taps), init="norm", role="vector"),
            n["k_conv"]: TensorSpec((gd, taps), init="norm", role="vector"),
            n["v_conv"]: TensorSpec((hv, taps), init="norm", role="vector"),
            n["beta"]: TensorSpec((H, W)),
            n["A_log"]: TensorSpec((H,), init="zeros", role="vector"),
            n["norm"]: TensorSpec((self.value_dim,), init="norm", role="vector"),
            n["o"]: TensorSpec((W, hv)),
        }
        if self.channel_decay:
            specs[n["a1"]] = TensorSpec((self.decay_rank, W))
            specs[n["a2"]] = TensorSpec((H * self.head_dim, self.decay_rank))
            specs[n["dt_bias"]] = TensorSpec((H * self.head_dim,), init="zeros", role="vector")
        else:
            specs[n["decay"]] = TensorSpec((H, W))
            specs[n["dt_bias"]] = TensorSpec((H,), init="zeros", role="vector")
        if self.low_rank_gate:
            specs[n["g1"]] = TensorSpec((self.gate_rank, W))
            specs[n["g2"]] = TensorSpec((hv, self.gate_rank))
        else:
            specs[n["g"]] = TensorSpec((hv, W))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = {key: tensors[name] for key, name in self.names.items() if name in tensors}
        # the joined projection's rows: q, k, v, beta, then what makes the decay, then what makes the gate
        decay_rows = t["a1"] if self.channel_decay else t["decay"]
        gate_rows = t["g1"] if self.low_rank_gate else t["g"]
        if self.channel_decay and t["a1"].shape[0] != t["a2"].shape[1]:
            raise ValueError(f"{self.prefix}: the decay's two matrices do not fit each other: "
                             f"{tuple(t['a1'].shape)} and {tuple(t['a2'].shape)}")
        if self.low_rank_gate and t["g1"].shape[0] != t["g2"].shape[1]:
            raise ValueError(f"{self.prefix}: the gate's two matrices do not fit each other: "
                             f"{tuple(t['g1'].shape)} and {tuple(t['g2'].shape)}")
        self._w_in = torch.cat([t["q"], t["k"], t["v"], t["beta"], decay_rows, gate_rows], dim=0).contiguous()
        self._w_out = t["o"]
        self.beta_off = self.conv_channels
        self.decay_off = self.beta_off + self.num_heads
        self.decay_cols = int(decay_rows.shape[0])
        self.g_off = self.decay_off + self.decay_cols
        self.gate_cols = int(gate_rows.shape[0])
        # decays per channel are formed in 32-bit: the low-rank projection's second matrix multiplies in fp32
        self.a2 = t["a2"].contiguous() if self.channel_decay else None
        self.g2 = None
        if self.low_rank_gate:
            from .linear import Linear
            self.g2 = Linear(t["g2"])
        self.conv_weight = torch.cat([t["q_conv"], t["k_conv"], t["v_conv"]], dim=0).float().contiguous()
        self.a_log, self.dt_bias = t["A_log"].float().contiguous(), t["dt_bias"].float().contiguous()
        self.norm_weight = t["norm"].float().contiguous()
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def state_elements(self) -> int:
        # S of every head, then the convolution's last inputs
        return self.num_heads * self.head_dim * self.value_dim + self.conv_channels * (self.conv_taps - 1)

    def activation_elements(self) -> int:
        return 3 * self.conv_channels + 4 * self.inner_width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, T = ctx.batch, y.shape[0]
        s_elems = self.num_heads * self.head_dim * self.value_dim
        qkv = torch.empty((T, self.conv_channels), dtype=torch.float32, device=y.device)
        K.causal_conv_act(y, col0, self.conv_weight, qkv, ctx.state, state_off + s_elems, batch.entry_q_start,
                          batch.entry_seat, batch.max_q_len)
        o = torch.empty((T, self.inner_width), dtype=torch.float32, device=y.device)
        if self.channel_decay:
            # bias, softplus, the head's rate and the exponential in the second product's epilogue
            d0 = col0 + self.decay_off
            g = K.small_product_f32(y[:, d0:d0 + self.decay_cols], self.a2,
                                    torch.empty((T, self.num_heads * self.head_dim), dtype=torch.float32, device=y.device),
                                    bias=self.dt_bias, rate_log=self.a_log)
            K.gated_delta_rule(qkv, y, col0 + self.beta_off, 0, None, None, o, ctx.state, state_off,
                               batch.entry_q_start, batch.entry_seat, self.num_heads, self.num_kv_heads,
                               self.head_dim, self.value_dim, self.unit_eps, channel_decay=g)
        else:
            K.gated_delta_rule(qkv, y, col0 + self.beta_off, col0 + self.decay_off, self.a_log, self.dt_bias, o,
                               ctx.state, state_off, batch.entry_q_start, batch.entry_seat, self.num_heads,
                               self.num_kv_heads, self.head_dim, self.value_dim, self.unit_eps)
        if self.low_rank_gate:
            g0 = col0 + self.g_off
            gate, gate_off = self.g2(y[:, g0:g0 + self.gate_cols].contiguous()), 0
        else:
            gate, gate_off = y, col0 + self.g_off
        K.head_norm_gate(o, self.norm_weight, self.norm_eps, gate, gate_off, out, out_col0, self.num_heads,
                         self.value_dim, self.gate, mul)


@MIXERS.register("lightning_attention")
class LightningAttention(ProjectedMixer):
    """Linear attention with one fixed decay a head: ``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T
    (query_scale q_t)`` where q, k and v are the ``activation`` (silu) of their projections.  The heads'
    read-outs are normed TOGETHER (one RMS norm over ``heads * value_dim`` elements with a weight of
    that size), gated element by element with ``gate(W_g x)`` and projected.  The decays are
    constants of the model, not tensors.  State: ``S`` of every head, fp32."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay,
                 norm_eps: float, query_scale: float = 1.0, activation: Optional[str] = "silu", gate: str = "sigmoid",
                 tensor_names: Optional[Dict[str, str]] = None):
        """``decay``: one number a head.  ``tensor_names`` maps ``q k v g o norm`` to names behind ``prefix``."""
        super().__init__(prefix)
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.decay = tuple(float(a) for a in decay)
        if len(self.decay) != self.num_heads:
            raise ValueError(f"{prefix}: {len(self.decay)} decays for {self.num_heads} heads")
        if gate not in K.HEAD_GATES:
            raise ValueError(f"{prefix}: gate {gate!r} is not one of {sorted(K.HEAD_GATES)}")
        self.norm_eps, self.query_scale, self.activation, self.gate = float(norm_eps), float(query_scale), activation, gate
        self.inner_width = self.num_heads * self.value_dim
        self.names = _names(dict(q="q", k="k", v="v", g="g", o="o", norm="norm"), tensor_names, prefix)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, hd, hv = self.names, self.hidden_size, self.num_heads * self.head_dim, self.inner_width
        return {n["q"]: TensorSpec((hd, W)), n["k"]: TensorSpec((hd, W)), n["v"]: TensorSpec((hv, W)),
                n["g"]: TensorSpec((hv, W)), n["o"]: TensorSpec((W, hv)),
                n["norm"]: TensorSpec((hv,), init="norm", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = {key: tensors[name] for key, name in self.names.items()}
        self._w_in = torch.cat([t["q"], t["k"], t["v"], t["g"]], dim=0).contiguous()
        self._w_out = t["o"]
        hd, hv = self.num_heads * self.head_dim, self.inner_width
        self.q_off, self.k_off, self.v_off, self.g_off = 0, hd, 2 * hd, 2 * hd + hv
        self.norm_weight = t["norm"].float().contiguous()
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=self._w_in.device)
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def state_elements(self) -> int:
        return self.num_heads * self.head_dim * self.value_dim

    def activation_elements(self) -> int:
        return 2 * self.num_heads * self.head_dim + 5 * self.inner_width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, T = ctx.batch, y.shape[0]
        o = torch.empty((T, self.inner_width), dtype=torch.float32, device=y.device)
        K.gated_linear_attention(y, col0 + self.q_off, col0 + self.k_off, col0 + self.v_off, None, self.query_scale, o,
                                 ctx.state, state_off, batch.entry_q_start, batch.entry_seat, self.num_heads,
                                 self.head_dim, self.value_dim, head_decay=self.head_decay, activation=self.activation)
        # one norm over all the heads' read-outs: a single "head" as wide as the row
        K.head_norm_gate(o, self.norm_weight, self.norm_eps, y, col0 + self.g_off, out, out_col0, 1, self.inner_width,
                         self.gate, mul)


@MIXERS.register("matrix_memory")
class MatrixMemory(ProjectedMixer):
    """A matrix memory with exponential gates.  Per head: ``q = W_q x * query_scale`` (default ``head_dim^-1/2``),
    ``k = W_k x`` (``head_dim``), ``v = W_v x`` (``value_dim``); a log input gate ``i = cap tanh((W_i x + b_i) /
    cap)`` and a log forget gate ``f = logsigmoid(cap tanh((W_f x + b_f) / cap))``; with a running maximum m
    (0 at a request's start, like S and n): ``m' = max(f + m, i)``, ``S <- e^(f + m - m') S + e^(i - m') k v^T``,
    ``n <- e^(f + m - m') n + e^(i - m') k``, ``o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)``.  Every head's
    read-out is divided by its root mean square, the heads are joined and multiplied by a weight of all
    heads' size and by ``gate(W_g x)``, then projected.  The gates' inputs are formed in 32-bit from the
    mixer's input rows (a product of their own, not columns of the joined projection); S, n and m are fp32
    in the seat's state row."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, gate_cap: float,
                 norm_eps: float, query_scale: Optional[float] = None, gate: str = "sigmoid",
                 tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``q k v g o norm i f i_bias f_bias`` to names behind ``prefix``."""
        super().__init__(prefix)
        if gate not in K.HEAD_GATES:
            raise ValueError(f"{prefix}: gate {gate!r} is not one of {sorted(K.HEAD_GATES)}")
        if not gate_cap > 0:
            raise ValueError(f"{prefix}: gate_cap {gate_cap} must be positive")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.gate_cap, self.norm_eps, self.gate = float(gate_cap), float(norm_eps), gate
        self.query_scale = float(head_dim) ** -0.5 if query_scale is None else float(query_scale)
        self.inner_width = self.num_heads * self.value_dim
        self.names = _names(dict(q="q", k="k", v="v", g="g", o="o", norm="norm", i="i", f="f", i_bias="i.b", f_bias="f.b"),
                            tensor_names, prefix)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, H, hd, hv = self.names, self.hidden_size, self.num_heads, self.num_heads * self.head_dim, self.inner_width
        return {n["q"]: TensorSpec((hd, W)), n["k"]: TensorSpec((hd, W)), n["v"]: TensorSpec((hv, W)),
                n["g"]: TensorSpec((hv, W)), n["o"]: TensorSpec((W, hv)),
                n["norm"]: TensorSpec((hv,), init="norm", role="vector"),
                n["i"]: TensorSpec((H, W)), n["f"]: TensorSpec((H, W)),
                n["i_bias"]: TensorSpec((H,), init="normal", role="vector"),
                n["f_bias"]: TensorSpec((H,), init="normal", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = {key: tensors[name] for key, name in self.names.items()}
        self._w_in = torch.cat([t["q"], t["k"], t["v"], t["g"]], dim=0).contiguous()
        self._w_out = t["o"]
        hd, hv = self.num_heads * self.head_dim, self.inner_width
        self.q_off, self.k_off, self.v_off, self.g_off = 0, hd, 2 * hd, 2 * hd + hv
        self.gate_weight = torch.cat([t["i"], t["f"]], dim=0).contiguous()                     # [2 heads, hidden]: zi, then zf
        self.gate_bias = torch.cat([t["i_bias"], t["f_bias"]]).float().contiguous()
        self.norm_weight = t["norm"].float().contiguous()
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def state_elements(self) -> int:
        # S of every head, then n and m as the kernel lays them out (a copy per run of 16 value columns)
        tiles = -(-self.value_dim // 16)
        return self.num_heads * self.head_dim * self.value_dim + self.num_heads * tiles * (self.head_dim + 1)

    def activation_elements(self) -> int:
        return 2 * self.num_heads * self.head_dim + 5 * self.inner_width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, T = ctx.batch, y.shape[0]
        if ctx.x is None:
            raise K.KernelError(f"{self.prefix}: the gates are formed from the mixer's input rows, which were not handed on")
        if self.state_elements() != K.matrix_memory_state(self.num_heads, self.head_dim, self.value_dim):
            raise K.KernelError(f"{self.prefix}: the kernel lays the state out differently")
        gates = K.small_product_f32(ctx.x, self.gate_weight,
                                    torch.empty((T, 2 * self.num_heads), dtype=torch.float32, device=y.device),
                                    bias=self.gate_bias)
        o = torch.empty((T, self.inner_width), dtype=torch.float32, device=y.device)
        K.matrix_memory(y, col0 + self.q_off, col0 + self.k_off, col0 + self.v_off, gates, self.gate_cap, self.query_scale,
                        o, ctx.state, state_off, batch.entry_q_start, batch.entry_seat, self.num_heads, self.head_dim,
                        self.value_dim)
        K.head_norm_gate(o, self.norm_weight, self.norm_eps, y, col0 + self.g_off, out, out_col0, self.num_heads,
                         self.value_dim, self.gate, mul)


@MIXERS.register("real_gated_lru")
class RealGatedLRU(ProjectedMixer):
    """A recurrent block around a real-gated linear recurrent unit.  Two branches of ``width`` channels read
    the input: ``y = gelu_tanh(W_y x + b_y)`` and ``u = conv(W_x x + b_x)``, a causal convolution per channel
    over ``conv_taps`` tokens (weight ``[channels, taps]``, the last column the current token's; a bias; no
    activation; zeros before a request's start).  The channels come in ``blocks`` equal runs; in run b ``r =
    sigmoid(A_b u_b + a_b)`` and ``i = sigmoid(B_b u_b + b_b)`` with square matrices ``[out, in]``.  Then ``log a
    = -rate_scale * r * softplus(lam)``, ``S_t = a S_(t-1) + sqrt(1 - a^2) i u`` (from ``S = 0``, the first
    token like every other), and the output projection reads ``S * y``.  Everything behind the convolution
    is fp32; the state row holds S and then the convolution's last ``taps - 1`` inputs."""

    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, width: int, blocks: int, conv_taps: int, rate_scale: float = 8.0,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``y x y_bias x_bias conv conv_bias a i a_bias i_bias lam o`` to names behind ``prefix``."""
        super().__init__(prefix)
        self.hidden_size, self.width, self.blocks, self.conv_taps = int(hidden_size), int(width), int(blocks), int(conv_taps)
        if self.blocks <= 0 or self.width % self.blocks:
            raise ValueError(f"{prefix}: {width} channels do not come in {blocks} equal runs")
        if not 1 <= self.conv_taps <= 17:
            raise ValueError(f"{prefix}: a convolution of {conv_taps} taps (1..17 are built)")
        self.rate_scale = float(rate_scale)
        self.inner_width = self.width
        self.names = _names(dict(y="y", x="x", y_bias="y.b", x_bias="x.b", conv="conv", conv_bias="conv.b", a="ra", i="ri",
                                 a_bias="ra.b", i_bias="ri.b", lam="lam", o="o"), tensor_names, prefix)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, C, B = self.names, self.hidden_size, self.width, self.blocks
        bs = C // B
        vec = dict(init="normal", role="vector")
        return {n["y"]: TensorSpec((C, W)), n["x"]: TensorSpec((C, W)), n["y_bias"]: TensorSpec((C,), **vec),
                n["x_bias"]: TensorSpec((C,), **vec), n["conv"]: TensorSpec((C, self.conv_taps), init="norm", role="vector"),
                n["conv_bias"]: TensorSpec((C,), **vec), n["a"]: TensorSpec((B, bs, bs)), n["i"]: TensorSpec((B, bs, bs)),
                n["a_bias"]: TensorSpec((B, bs), **vec), n["i_bias"]: TensorSpec((B, bs), **vec),
                n["lam"]: TensorSpec((C,), init="norm", role="vector"), n["o"]: TensorSpec((W, C))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = {key: tensors[name] for key, name in self.names.items()}
        self._w_in = torch.cat([t["y"], t["x"]], dim=0).contiguous()
        self._w_out = t["o"]
        self.y_off, self.x_off = 0, self.width
        self.y_bias, self.x_bias = t["y_bias"].float().contiguous(), t["x_bias"].float().contiguous()
        self.conv_weight, self.conv_bias = t["conv"].float().contiguous(), t["conv_bias"].float().contiguous()
        self.w_a, self.w_i = t["a"].contiguous(), t["i"].contiguous()
        self.a_bias, self.i_bias = t["a_bias"].float().reshape(-1).contiguous(), t["i_bias"].float().reshape(-1).contiguous()
        # the decay's rate per channel, rate_scale * softplus(lam): a constant of the weights, formed once in 32-bit
        self.rate = (self.rate_scale * torch.nn.functional.softplus(t["lam"].float())).contiguous()
        self.load_projections()

    def input_weight(self) -> torch.Tensor:
        return self._w_in

    def output_weight(self) -> torch.Tensor:
        return self._w_out

    def state_elements(self) -> int:
        return self.width * self.conv_taps          # S, then taps - 1 inputs per channel

    def activation_elements(self) -> int:
        return 2 * self.width + 3 * 2 * self.width + self.width + self.hidden_size

    def forward_inner(self, y, col0, ctx: MixerContext, state_off, out, out_col0, mul) -> None:
        batch, T = ctx.batch, y.shape[0]
        u = torch.empty((T, self.width), dtype=torch.float32, device=y.device)
        K.causal_conv_act(y, col0 + self.x_off, self.conv_weight, u, ctx.state, state_off + self.width, batch.entry_q_start,
                          batch.entry_seat, batch.max_q_len, in_bias=self.x_bias, out_bias=self.conv_bias, activation=None)
        a, b = torch.empty_like(u), torch.empty_like(u)
        K.block_gates(u, self.w_a, self.w_i, self.a_bias, self.i_bias, self.rate, a, b)
        K.linear_scan_gate(a, b, y, col0 + self.y_off, self.y_bias, out, out_col0, ctx.state, state_off,
                           batch.entry_q_start, batch.entry_seat, mul)
