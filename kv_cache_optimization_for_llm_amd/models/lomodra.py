"""The Lomodra decoder as data: its ``config.json`` -> ModelSpec.

A decoder over a residual stream kept in 32-bit whose branches read the stream ITSELF and whose
norms (RMS, plain weight) stand on the branches' outputs: ``x += n1(mixer(x)); x += n2(ff(x))``.
After the feed-forward every layer adds something the token brings along: its own ``dim`` columns
``e`` of a second embedding table, gated and projected, ``x += n3(W_proj (gelu(W_gate x) * e))``.
A layer's mixer is

* ``lightning``: linear attention with one fixed decay a head (a constant of the model), silu on
  q, k, v, one norm over all heads' read-outs, a sigmoid gate;
* ``attention``: grouped-query softmax attention without positions in the scores, queries and keys
  under an RMS norm per head, visible keys confined to the query's own chunk of ``mask.size``
  positions; with ``kv_from: j`` the layer has no keys and values of its own and attends over
  those layer j wrote;
* ``channel_delta``: a gated delta rule with short convolutions whose decay has one value per head
  and key channel (a low-rank projection), and a low-rank sigmoid output gate.

The feed-forward is a mixture of gated silu experts - router logits with a bias, the largest
``top`` chosen, weights a softmax over the chosen logits - plus one expert that every token uses; or
absent.  The model's norm at the end, logits from the token table itself, then a soft cap.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from .gadopel import _need
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

LAYER_TYPES = ("lightning", "attention", "channel_delta")
FEED_FORWARD_KINDS = ("moe",)


def _positive(m: Mapping[str, Any], keys, where: str) -> None:
    for key in keys:
        if _need(m, key, where) <= 0:
            raise ConfigError(f"config.json: {where}.{key} must be positive")


def _kv_heads(m: Mapping[str, Any], where: str) -> None:
    g = _need(m, "kv_heads", where)
    if g <= 0 or m["heads"] % g:
        raise ConfigError(f"config.json: {where}: {m['heads']} heads is not a multiple of {g} kv heads")


def _check_mixer(kind: str, m: Mapping[str, Any], where: str, index: int, layers) -> None:
    if kind == "attention" and isinstance(m, dict) and isinstance(m.get("kv_from"), int) and 0 <= m["kv_from"] < index:
        # sizes of keys and values that such a layer leaves out are those of the layer it takes them from
        om = layers[m["kv_from"]].get("mixer") if isinstance(layers[m["kv_from"]], Mapping) else None
        for key in ("kv_heads", "dim", "vdim"):
            if key not in m and isinstance(om, Mapping) and key in om:
                m[key] = om[key]
    _positive(m, ("heads", "dim", "vdim"), where)
    if kind == "lightning":
        decay = m.get("decay")
        if not isinstance(decay, (list, tuple)) or len(decay) != m["heads"] \
                or any(isinstance(a, bool) or not isinstance(a, (int, float)) for a in decay):
            raise ConfigError(f"config.json: {where}.decay must list one number for each of the {m['heads']} heads")
        return
    _kv_heads(m, where)
    if kind == "channel_delta":
        if not 1 <= _need(m, "conv", where) <= 17:
            raise ConfigError(f"config.json: {where}.conv must lie in 1..17")
        return
    _need(m, "scale", where, float)
    if m["dim"] % 4:
        raise ConfigError(f"config.json: {where}.dim {m['dim']} must be a multiple of 4 (keys lie in the cache in "
                          "chunks of 4 or 8 elements)")
    if m.get("mask") is not None and _need(m["mask"], "size", where + ".mask") <= 0:
        raise ConfigError(f"config.json: {where}.mask.size must be positive")
    j = m.get("kv_from")
    if j is not None:
        if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < index:
            raise ConfigError(f"config.json: {where}.kv_from must name an earlier layer")
        other = layers[j]
        om = other.get("mixer") if isinstance(other, Mapping) else None
        if other.get("type") != "attention" or not isinstance(om, Mapping) or om.get("kv_from") is not None:
            raise ConfigError(f"config.json: {where}.kv_from = {j}: that layer has no keys and values of its own")
        if any(om.get(key) != m.get(key) for key in ("kv_heads", "dim", "vdim")):
            raise ConfigError(f"config.json: {where}.kv_from = {j}: the two layers' key and value sizes differ")


def _check_mlp(mlp: Mapping[str, Any], where: str) -> None:
    if mlp.get("kind") not in FEED_FORWARD_KINDS:
        raise ConfigError(f"config.json: {where}.kind must be one of {FEED_FORWARD_KINDS}")
    _positive(mlp.get("expert"), ("ff",), where + ".expert")
    r = mlp.get("router")
    experts, top = _need(r, "experts", where + ".router"), _need(r, "top", where + ".router")
    if not 0 < top <= experts:
        raise ConfigError(f"config.json: {where}.router: top {top} of {experts} experts")
    if mlp.get("shared") is not None:
        _positive(mlp["shared"], ("ff",), where + ".shared")


@dataclass(frozen=True)
class LomodraConfig:
    """``config.json`` of a Lomodra model, checked: ``vocab``, ``width``, ``norm.eps``, ``logit_softcap``,
    ``token_side.dim`` (or no ``token_side``) and ``layers`` (per layer ``type``, ``mixer``, ``mlp`` or null)."""

    vocab: int
    width: int
    norm_eps: float
    logit_softcap: float
    side_dim: int
    layers: Tuple[Mapping[str, Any], ...]
    max_positions: int

    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "LomodraConfig":
        vocab, width = _need(d, "vocab", "the model"), _need(d, "width", "the model")
        if vocab <= 0 or width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        eps = _need(d.get("norm"), "eps", "norm", float)
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = copy.deepcopy(list(layers))      # (sizes a layer inherits are filled in below; the caller's dict stays)
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type must be one of {LAYER_TYPES}")
            _check_mixer(layer["type"], layer.get("mixer"), where + ".mixer", i, layers)
            if layer.get("mlp") is not None:
                _check_mlp(layer["mlp"], where + ".mlp")
        cap = d.get("logit_softcap")
        cap = 0.0 if cap is None else _need(d, "logit_softcap", "the model", float)
        if cap < 0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        side = d.get("token_side")
        side_dim = 0 if side is None else _need(side, "dim", "token_side")
        if side is not None and side_dim <= 0:
            raise ConfigError("config.json: token_side.dim must be positive")
        return LomodraConfig(vocab=vocab, width=width, norm_eps=eps, logit_softcap=cap, side_dim=side_dim,
                             layers=tuple(layers), max_positions=int(d.get("max_positions", 1 << 17)))


def _norm(prefix: str, name: str, width: int, eps: float) -> PartSpec:
    # an RMS norm that reads or feeds a 32-bit stream whatever the products' type is
    return PartSpec("layernorm", dict(prefix=prefix, width=width, eps=eps, weight_name=name, center=False))


def _mixer(kind: str, m: Mapping[str, Any], p: str, W: int, eps: float) -> PartSpec:
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    if kind == "lightning":
        return PartSpec("lightning_attention", dict(
            prefix=p, hidden_size=W, num_heads=H, head_dim=d, value_dim=dv, decay=tuple(float(a) for a in m["decay"]),
            norm_eps=eps, query_scale=1.0, activation="silu", gate="sigmoid"))
    if kind == "channel_delta":
        return PartSpec("gated_delta_rule", dict(
            prefix=p, hidden_size=W, num_heads=H, num_kv_heads=int(m["kv_heads"]), head_dim=d, value_dim=dv,
            conv_taps=int(m["conv"]), norm_eps=eps, unit_eps=1e-6, decay="channel", decay_rank=m.get("decay_rank"),
            gate="sigmoid", low_rank_gate=True, gate_rank=m.get("gate_rank")))
    mask = m.get("mask") or {}
    return PartSpec("normed_gqa_attention", dict(
        prefix=p, hidden_size=W, num_heads=H, num_kv_heads=int(m["kv_heads"]), head_dim=d, value_dim=dv,
        scale=float(m["scale"]), norm_eps=eps, chunk=int(mask.get("size", 0) or 0), shared_kv=m.get("kv_from") is not None))


def lomodra_spec(cfg: LomodraConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        norms = {"mixer": _norm(p, "norm1", W, eps)}
        mlp = layer.get("mlp")
        if mlp is not None:
            r, shared = mlp["router"], mlp.get("shared")
            ffn = PartSpec("routed_experts", dict(
                prefix=p + "mlp.", hidden_size=W, intermediate_size=int(mlp["expert"]["ff"]), experts=int(r["experts"]),
                top=int(r["top"]), activation="silu", correction=False, gated=True, router_bias=True,
                softmax_over="chosen", shared_intermediate=int(shared["ff"]) if shared is not None else 0))
            norms["feed_forward"] = _norm(p, "norm2", W, eps)
        else:
            ffn = PartSpec("none")
        block = {}
        if cfg.side_dim:
            block["layer_input"] = PartSpec("gated_table", dict(
                prefix=p + "side.", hidden_size=W, dim=cfg.side_dim, table_name="side.embed", table_rows=cfg.vocab,
                table_width=len(cfg.layers) * cfg.side_dim, column=i * cfg.side_dim, eps=eps, activation="gelu_tanh"))
        layers.append(LayerSpec(block=PartSpec("post_norm", block), mixer=_mixer(layer["type"], m, p + "mix.", W, eps),
                                feed_forward=ffn, norms=norms, prefix=p))
        j = m.get("kv_from") if layer["type"] == "attention" else None
        # a layer that takes another layer's keys and values reads that layer's cache slot and writes nothing
        order.append(LayerCall(layer=i, cache=i if j is None else int(j), writes_cache=j is None))
    ignorable = tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None)
    return ModelSpec(
        architecture="Lomodra", hidden_size=W, vocab_size=cfg.vocab, embedding_name="embed",
        layers=tuple(layers), order=tuple(order), final_norm=_norm("final.", "norm", W, eps),
        final_norm_prefix="final.", head_name=None, max_positions=cfg.max_positions,
        logit_softcap=cfg.logit_softcap, residual_dtype="float32", ignorable_tensors=ignorable)


register_architecture("Lomodra", LomodraConfig.from_dict, lomodra_spec, replace=True)
