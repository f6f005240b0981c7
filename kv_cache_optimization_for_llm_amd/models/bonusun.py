"""The Bonusun decoder as data: its ``config.json`` -> ModelSpec.

A pre-norm decoder over a residual stream kept in 32-bit whose norms are layer norms with weight
and bias and whose branches enter the stream times a constant, ``x += m * branch(norm(x))`` - or,
with ``streams``, through hyper-connections: the stream is several copies of every row, a branch
reads a weighted sum of them, and its output re-enters all of them at once beside a mixing of the
old copies.  A layer's mixer is

* ``attention``: grouped-query softmax attention with an RMS norm per head on queries and keys
  (before the rotation), a rotate-half rotation of a head's first elements (optionally with every
  frequency divided by a factor), an optional sliding window, a value size of its own and a sink
  per head in the softmax's denominator;
* ``parallel``: such an attention (``left``) beside a matrix memory with exponential gates
  (``right``) on the same input, added with two constants;
* ``rglru``: a real-gated linear recurrent unit behind a short causal convolution, times a gelu
  branch.

Its feed-forward is dense (``down(gelu_tanh(up(x)))``), a mixture of clamped gated experts under
a sigmoid router that chooses inside the best groups of experts, beside an expert every token uses
under a gate of its own, or absent.  A run of layers may be repeated with the same weights, every
pass over a cache and state of its own.  Layer norm at the end (over the sum of the copies), then
the output matrix ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from .gadopel import _need
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

LAYER_TYPES = ("attention", "parallel", "rglru")
FEED_FORWARD_KINDS = ("dense", "moe")
# constants the design fixes
RGLRU_RATE = 8.0            # log a = -8 r softplus(lam)
GROUP_TOP = 2               # a group of experts is scored by its two largest choice scores
WEIGHT_SUM_EPS = 1e-20      # added to the sum the chosen experts' scores are divided by
MAX_STREAMS = 8


def _check_attention(m: Mapping[str, Any], where: str) -> None:
    for key in ("heads", "kv_heads", "dim", "vdim"):
        if _need(m, key, where) <= 0:
            raise ConfigError(f"config.json: {where}.{key} must be positive")
    if m["heads"] % m["kv_heads"]:
        raise ConfigError(f"config.json: {where}: {m['heads']} heads is not a multiple of {m['kv_heads']} kv heads")
    if m["dim"] % 4:
        raise ConfigError(f"config.json: {where}.dim {m['dim']} must be a multiple of 4 (keys lie in the cache in "
                          "chunks of 4 or 8 elements)")
    _need(m, "scale", where, float)
    rot = m.get("rot")
    if rot is not None:
        dims = _need(rot, "dims", where + ".rot")
        if _need(rot, "base", where + ".rot", float) <= 0:
            raise ConfigError(f"config.json: {where}.rot.base must be positive")
        if dims % 2 or not 0 <= dims <= m["dim"]:
            raise ConfigError(f"config.json: {where}.rot.dims {dims} must be even and at most dim {m['dim']}")
        if rot.get("scaling") is not None and _need(rot["scaling"], "factor", where + ".rot.scaling", float) <= 0:
            raise ConfigError(f"config.json: {where}.rot.scaling.factor must be positive")
    if m.get("mask") is not None and _need(m["mask"], "size", where + ".mask") <= 0:
        raise ConfigError(f"config.json: {where}.mask.size must be positive")


def _check_mixer(kind: str, m: Mapping[str, Any], where: str) -> None:
    if not isinstance(m, Mapping):
        raise ConfigError(f"config.json: {where} must give the mixer's sizes")
    if kind == "attention":
        _check_attention(m, where)
    elif kind == "parallel":
        _check_attention(m.get("left"), where + ".left")
        right = m.get("right")
        for key in ("heads", "dim", "vdim"):
            if _need(right, key, where + ".right") <= 0:
                raise ConfigError(f"config.json: {where}.right.{key} must be positive")
        if _need(right, "gate_cap", where + ".right", float) <= 0:
            raise ConfigError(f"config.json: {where}.right.gate_cap must be positive")
        _need(m, "left_scale", where, float)
        _need(m, "right_scale", where, float)
    else:
        width, blocks = _need(m, "width", where), _need(m, "blocks", where)
        if width <= 0 or blocks <= 0 or width % blocks:
            raise ConfigError(f"config.json: {where}: {width} channels do not come in {blocks} equal parts")
        if not 1 <= _need(m, "conv", where) <= 17:
            raise ConfigError(f"config.json: {where}.conv must lie in 1..17")


def _check_mlp(mlp: Mapping[str, Any], where: str) -> None:
    if not isinstance(mlp, Mapping) or mlp.get("kind") not in FEED_FORWARD_KINDS:
        raise ConfigError(f"config.json: {where}.kind must be one of {FEED_FORWARD_KINDS}")
    if mlp["kind"] == "dense":
        if _need(mlp, "ff", where) <= 0:
            raise ConfigError(f"config.json: {where}.ff must be positive")
        return
    if _need(mlp.get("expert"), "ff", where + ".expert") <= 0:
        raise ConfigError(f"config.json: {where}.expert.ff must be positive")
    _need(mlp["expert"], "limit", where + ".expert", float)
    r = mlp.get("router")
    experts, top = _need(r, "experts", where + ".router"), _need(r, "top", where + ".router")
    if not 0 < top <= experts:
        raise ConfigError(f"config.json: {where}.router: top {top} of {experts} experts")
    if r.get("scale") is not None:
        _need(r, "scale", where + ".router", float)
    g = r.get("groups")
    if g is not None:
        count, keep = _need(g, "count", where + ".router.groups"), _need(g, "keep", where + ".router.groups")
        if count <= 0 or experts % count or not 0 < keep <= count or top > keep * (experts // count):
            raise ConfigError(f"config.json: {where}.router.groups: {count} groups of which {keep} are kept do not fit "
                              f"top {top} of {experts} experts")
    shared = mlp.get("shared")
    if shared is not None:
        if _need(shared, "ff", where + ".shared") <= 0:
            raise ConfigError(f"config.json: {where}.shared.ff must be positive")
        _need(shared, "limit", where + ".shared", float)


@dataclass(frozen=True)
class BonusunConfig:
    """``config.json`` of a Bonusun model, checked: ``vocab``, ``width``, ``norm.eps``, ``residual_mult``,
    ``streams`` (absent: one plain stream), ``layers`` (per layer ``type``, ``mixer`` and ``mlp`` or null)
    and the optional ``loop`` (``start``, ``stop``, ``times``)."""

    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    streams: Optional[int]
    layers: Tuple[Mapping[str, Any], ...]
    loop: Optional[Tuple[int, int, int]]
    max_positions: int

    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "BonusunConfig":
        vocab, width = _need(d, "vocab", "the model"), _need(d, "width", "the model")
        if vocab <= 0 or width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        eps = _need(d.get("norm"), "eps", "norm", float)
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type must be one of {LAYER_TYPES}")
            _check_mixer(layer["type"], layer.get("mixer"), where + ".mixer")
            if layer.get("mlp") is not None:
                _check_mlp(layer["mlp"], where + ".mlp")
        streams = d.get("streams")
        if streams is not None and not 1 <= _need(d, "streams", "the model") <= MAX_STREAMS:
            raise ConfigError(f"config.json: streams must lie in 1..{MAX_STREAMS}")
        loop = d.get("loop")
        if loop is not None:
            a, b, n = (_need(loop, k, "loop") for k in ("start", "stop", "times"))
            if not (0 <= a < b <= len(layers)) or n < 1:
                raise ConfigError(f"config.json: loop {a}..{b} x {n} does not fit {len(layers)} layers")
            loop = (a, b, n)
        mult = 1.0 if d.get("residual_mult") is None else _need(d, "residual_mult", "the model", float)
        return BonusunConfig(vocab=vocab, width=width, norm_eps=eps, residual_mult=mult, streams=streams,
                             layers=tuple(layers), loop=loop, max_positions=int(d.get("max_positions", 1 << 17)))


def _norm(prefix: str, name: str, width: int, eps: float, streams: int = 1) -> PartSpec:
    return PartSpec("layernorm", dict(prefix=prefix, width=width, eps=eps, weight_name=name, bias_name=name + ".b",
                                      streams=streams))


def _attention(m: Mapping[str, Any], p: str, W: int, eps: float, max_positions: int) -> PartSpec:
    rot = m.get("rot")
    if rot is not None and int(rot["dims"]) > 0:
        scaling = rot.get("scaling")
        rule = dict(frequencies="plain_f64") if scaling is None else \
            dict(frequencies="linear_f64", frequency_params=dict(factor=float(scaling["factor"])))
        position = PartSpec("rotary", dict(head_dim=int(m["dim"]), rotary_dim=int(rot["dims"]), max_positions=max_positions,
                                           theta=float(rot["base"]), pairing="half", **rule))
    else:
        position = PartSpec("none")
    return PartSpec("gated_gqa_attention", dict(
        prefix=p, hidden_size=W, num_heads=int(m["heads"]), num_kv_heads=int(m["kv_heads"]), head_dim=int(m["dim"]),
        value_dim=int(m["vdim"]), scale=float(m["scale"]), position=position, window=int((m.get("mask") or {}).get("size", 0)),
        bias=False, gate=None, qk_norm="before_rotation", norm_eps=eps, sink=True))


def _mixer(kind: str, m: Mapping[str, Any], p: str, W: int, eps: float, max_positions: int) -> PartSpec:
    if kind == "attention":
        return _attention(m, p, W, eps, max_positions)
    if kind == "rglru":
        return PartSpec("real_gated_lru", dict(prefix=p, hidden_size=W, width=int(m["width"]), blocks=int(m["blocks"]),
                                               conv_taps=int(m["conv"]), rate_scale=RGLRU_RATE))
    right = m["right"]
    memory = PartSpec("matrix_memory", dict(
        prefix=p + "right.", hidden_size=W, num_heads=int(right["heads"]), head_dim=int(right["dim"]),
        value_dim=int(right["vdim"]), gate_cap=float(right["gate_cap"]), norm_eps=eps, gate="sigmoid"))
    return PartSpec("side_by_side", dict(prefix=p, hidden_size=W,
                                         children=(_attention(m["left"], p + "left.", W, eps, max_positions), memory),
                                         scales=(float(m["left_scale"]), float(m["right_scale"]))))


def _feed_forward(mlp: Optional[Mapping[str, Any]], p: str, W: int) -> PartSpec:
    if mlp is None:
        return PartSpec("none")
    if mlp["kind"] == "dense":
        return PartSpec("mlp", dict(prefix=p, hidden_size=W, intermediate_size=int(mlp["ff"]), activation="gelu_tanh"))
    r, shared = mlp["router"], mlp.get("shared")
    groups = r.get("groups") or {}
    return PartSpec("routed_experts", dict(
        prefix=p, hidden_size=W, intermediate_size=int(mlp["expert"]["ff"]), experts=int(r["experts"]), top=int(r["top"]),
        activation="swish_clamped", gated=True, limit=float(mlp["expert"]["limit"]), correction=True, renormalise=True,
        scores="sigmoid", groups=int(groups.get("count", 1)), keep_groups=int(groups.get("keep", 1)), group_top=GROUP_TOP,
        weight_scale=float(r["scale"]) if r.get("scale") is not None else 1.0, sum_eps=WEIGHT_SUM_EPS,
        shared_intermediate=int(shared["ff"]) if shared else 0,
        shared_limit=float(shared["limit"]) if shared else None, shared_gate=bool(shared)))


def bonusun_spec(cfg: BonusunConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    S = 1 if cfg.streams is None else int(cfg.streams)
    layers, ignorable = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        norms = {"mixer": _norm(p, "norm1", W, eps)}
        if layer.get("mlp") is not None:
            norms["feed_forward"] = _norm(p, "norm2", W, eps)
        else:
            ignorable += [p + "norm2", p + "norm2.b", p + "hc2.*"]
        layers.append(LayerSpec(
            block=PartSpec("hyper_connections", dict(prefix=p, streams=S, learned=cfg.streams is not None,
                                                     residual_mult=cfg.residual_mult)),
            mixer=_mixer(layer["type"], layer["mixer"], p + "mix.", W, eps, cfg.max_positions),
            feed_forward=_feed_forward(layer.get("mlp"), p + "mlp.", W), norms=norms, prefix=p))
    # run order: the layers before the loop, the looped run `times` times with the same weights (every pass
    # over cache and state slots of its own), then the rest
    n = len(layers)
    a, b, times = cfg.loop if cfg.loop is not None else (n, n, 0)
    runs = list(range(a)) + list(range(a, b)) * times + list(range(b, n))
    order = tuple(LayerCall(layer=i, cache=slot) for slot, i in enumerate(runs))
    return ModelSpec(
        architecture="Bonusun", hidden_size=W, vocab_size=cfg.vocab, embedding_name="embed", layers=tuple(layers),
        order=order, final_norm=_norm("final.", "norm", W, eps, streams=S), final_norm_prefix="final.", head_name="head",
        max_positions=cfg.max_positions, residual_dtype="float32", streams=S, ignorable_tensors=tuple(ignorable))


register_architecture("Bonusun", BonusunConfig.from_dict, bonusun_spec, replace=True)
