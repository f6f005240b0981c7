"""Small Lomodra configurations with seeded weights, and helpers that compare an engine's rows with
the plain implementation (``plain_lomodra``).  Stepping an engine through a schedule and the row error
are the ones the other architectures' tests use (``radilix_util``)."""
import json
import os
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

import plain_lomodra as plain
from radilix_util import moe_calls, prompt, row_error, run_steps  # noqa: F401  (re-exported for the tests)


def moe(experts, top, ff, shared=None):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": None if shared is None else {"ff": shared}}


def attention_layer(heads, kv_heads, dim, vdim, scale, chunk=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def lightning_layer(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def delta_layer(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank, mlp=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": decay_rank, "gate_rank": gate_rank}, "mlp": mlp}


# The layers' eps is large in these configurations on purpose.  A recurrence's read-out is divided by its
# own root mean square; at a request's first token it is one value vector times q . k, and with a small
# eps the sign of a q . k near zero decides the whole row: rounding to bfloat16 then moves such a row by
# any amount.  With eps of the order of the read-out the division is smooth, and an eps in the wrong
# place shows all the more.
#
# A: values smaller than keys; two attention layers that take the FIRST layer's keys and values, each with
#    a chunk size of its own (7 and none at all); chunks of 24 over pages of 16 or 8; three taps; a value
#    size of the delta rule that is no multiple of 16; layers without a feed-forward; a router whose every
#    expert is chosen; an expert every token uses in one layer only.
CFG_A = {"architecture": "Lomodra", "vocab": 211, "width": 96, "norm": {"eps": 0.05}, "logit_softcap": 9.0,
         "token_side": {"dim": 12}, "layers": [
             attention_layer(4, 2, 32, 16, 0.21, chunk=24, mlp=moe(5, 2, 48, shared=40)),
             lightning_layer(3, 16, 8, (0.5, 0.9, 0.99)),
             attention_layer(4, 2, 32, 16, 0.4, chunk=7, kv_from=0),
             delta_layer(4, 2, 16, 24, 3, 6, 5, mlp=moe(3, 3, 40)),
             attention_layer(4, 2, 32, 16, 0.15, kv_from=0, mlp=moe(4, 1, 24, shared=16))]}
# B: a width that is no multiple of 32, no per-layer token input, no soft cap; attention over all earlier
#    keys (no mask) with as many kv heads as heads, and one with chunks of ONE position (every token sees
#    itself alone); one tap (no convolution); a decay of exactly 1 and a single head; one choice per token.
CFG_B = {"architecture": "Lomodra", "vocab": 157, "width": 72, "norm": {"eps": 0.1}, "layers": [
    lightning_layer(5, 8, 12, (1.0, 0.3, 0.8, 0.95, 0.999), mlp=moe(2, 1, 24)),
    attention_layer(3, 3, 20, 20, 0.3, mlp=moe(4, 2, 16, shared=8)),
    delta_layer(2, 2, 8, 8, 1, 3, 4),
    attention_layer(2, 1, 16, 32, 0.25, chunk=1),
    lightning_layer(1, 24, 40, (0.9,), mlp=moe(2, 1, 24))]}
# C: sizes at which the bf16 engine takes its matrix-core kernels: heads of 64 and 128, four query heads a
#    kv head, values of 32 beside keys of 64, chunks of 32 and of 100 positions, a layer that sees all of another
#    layer's keys, experts over a width of 256.
CFG_C = {"architecture": "Lomodra", "vocab": 257, "width": 256, "norm": {"eps": 0.02}, "logit_softcap": 30.0,
         "token_side": {"dim": 32}, "layers": [
             delta_layer(4, 2, 64, 32, 2, 16, 8, mlp=moe(6, 2, 128, shared=64)),
             attention_layer(8, 2, 64, 64, 0.11, chunk=32, mlp=moe(8, 3, 64)),
             lightning_layer(2, 128, 64, (0.97, 0.7), mlp=moe(6, 2, 128, shared=64)),
             attention_layer(8, 2, 64, 64, 0.2, chunk=100, kv_from=1),
             attention_layer(4, 1, 64, 32, 0.125, chunk=48, mlp=moe(4, 4, 32, shared=96)),
             attention_layer(2, 1, 128, 128, 0.09, chunk=16, mlp=None),
             attention_layer(8, 2, 64, 64, 0.3, kv_from=1, mlp=moe(6, 2, 128))]}
# D: no layer keeps keys and values (the cache manager has no paged group); keys of 160 channels (the
#    recurrences' kernels that keep the state in LDS); a single expert.
CFG_D = {"architecture": "Lomodra", "vocab": 131, "width": 64, "norm": {"eps": 0.05}, "logit_softcap": 5.0,
         "token_side": {"dim": 1}, "layers": [
             delta_layer(2, 1, 160, 24, 4, 4, 2, mlp=moe(1, 1, 32, shared=32)),
             lightning_layer(2, 160, 12, (0.8, 0.6)),
             delta_layer(3, 3, 12, 12, 5, 2, 7, mlp=moe(3, 2, 16))]}
CONFIGS = {"A": (CFG_A, 5), "B": (CFG_B, 6), "C": (CFG_C, 7), "D": (CFG_D, 8)}


def write_model(folder: str, cfg: dict, seed: int, gain: float = 1.0, edit=None) -> Tuple[str, Dict[str, torch.Tensor]]:
    """A model folder with seeded weights: matrices N(0, gain / sqrt(in)); what the random-weights mode
    leaves at zero or near one is spread out here so that it weighs in (norm weights, convolution taps,
    decay rates and biases, the routers' biases).  ``edit(state)`` may change the tensors before they are
    stored.  Returns the folder and the tensors as stored."""
    from safetensors.torch import save_file
    from kv_cache_optimization_for_llm_amd.models.builder import tensor_specs_for_config
    from kv_cache_optimization_for_llm_amd.weights.random_init import random_state_dict

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    state = random_state_dict(tensor_specs_for_config(cfg), seed, torch.bfloat16, gain)
    g = torch.Generator().manual_seed(seed)

    def rnd(shape, std, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)
    for name, t in state.items():
        if name.endswith((".norm1", ".norm2", "side.norm", "q.norm", "k.norm", "mix.norm")) or name == "final.norm":
            state[name] = rnd(t.shape, 0.3, 1.0)
        elif name.endswith(".conv"):
            state[name] = rnd(t.shape, 0.6)
        elif name.endswith(".A_log"):
            state[name] = rnd(t.shape, 0.7, -1.0)
        elif name.endswith(".dt_bias"):
            state[name] = rnd(t.shape, 0.8)
        elif name.endswith("router.b"):
            state[name] = rnd(t.shape, 0.3)
        elif name == "side.embed":
            state[name] = rnd(t.shape, 1.0)
    if edit is not None:
        edit(state)
    save_file(state, os.path.join(folder, "model.safetensors"))
    return folder, state


TOLERANCE = {"float32": 2e-4, "bfloat16": 6e-2}
LIMITS: Dict[str, List[float]] = {}      # per request and position, where expected_rows found a row ill-conditioned
# a router's choice is the engine's to make where the plain implementation's own margin (a gap between
# two logits) is below this: the engine's input to the router carries its format's rounding - in
# bfloat16 that of every layer before it, which moves a row of the stream by a few percent and a
# logit of size 3 by about a tenth.  (What a router does wrong shows in 32-bit, where no gap is forgiven.)
CLOSE_CALL = {"float32": 1e-4, "bfloat16": 0.3}


def bf16_rounding(t):
    return t.to(torch.bfloat16).to(plain.F)


def expected_rows(cfg: dict, state: Dict[str, torch.Tensor], requests: Dict[str, List[int]], routes=None,
                  dtype: str = "float32", close_call: Optional[float] = None) -> Dict[str, np.ndarray]:
    """Logits of the plain forward pass per request.  With ``routes`` (what the engine's routers chose)
    the plain experts are the engine's, and every choice that differs from the plain router's own
    must be a close call of that router."""
    W = plain.to_f64(state)
    out = {}
    LIMITS.clear()
    for rid, toks in requests.items():
        forced = None
        if routes is not None:
            forced = {layer: idx[:len(toks)] for layer, idx in routes[rid].items()}
        margins: dict = {}
        out[rid] = plain.forward(cfg, W, toks, forced=forced, margins=margins).numpy()
        if dtype == "bfloat16":
            # the limit of a row is three times what rounding the projections' and the branches' outputs to
            # bfloat16 does to it in the plain model, where that is more than the general limit
            moved = plain.forward(cfg, W, toks, forced=forced, rounded=bf16_rounding).numpy()
            LIMITS[rid] = [max(TOLERANCE[dtype], 3.0 * row_error(moved[p], out[rid][p])) for p in range(len(toks))]
        if forced is not None:
            for layer, (own, margin) in margins.items():
                differs = (forced[layer].sort(-1).values != own.sort(-1).values).any(-1)
                assert (margin[differs] <= (CLOSE_CALL[dtype] if close_call is None else close_call)).all(), \
                    f"request {rid}, layer {layer}: the engine's router chose other experts where the choice was clear"
    return out


def assert_rows(rows, expected: Dict[str, np.ndarray], dtype: str, what: str = "") -> float:
    """Every row within its limit in 32-bit.  In bfloat16 a row's limit is an estimate (one sample of
    what rounding does at that place), so: no row beyond twice its limit, at most one in fifty (or one) beyond it."""
    worst, over = 0.0, 0
    for (rid, p), row in rows.items():
        assert np.isfinite(row).all(), f"{what}: request {rid} position {p} has a logit that is not finite"
        e = row_error(row, expected[rid][p])
        limit = LIMITS[rid][p] if dtype == "bfloat16" and rid in LIMITS else TOLERANCE[dtype]
        hard = 2.0 * limit if dtype == "bfloat16" else limit
        assert e <= hard, f"{what}: request {rid} position {p} is off by {e:.3g} (limit {hard:.3g})"
        over += e > limit
        worst = max(worst, e)
    assert over <= max(1, len(rows) // 50), f"{what}: {over} of {len(rows)} rows are beyond their limits"
    return worst
