"""The plain Bonusun (``plain_bonusun``) pinned against other formulations of its mechanisms, and the
configuration reader, the run order and the tensor names of the engine's description of the design.  No GPU."""
import copy
import math

import pytest
import torch

import bonusun_util as U
import plain_bonusun as plain
from kv_cache_optimization_for_llm_amd.config.model_config import ConfigError
from kv_cache_optimization_for_llm_amd.models.builder import spec_for_config, tensor_specs_for_config

F = plain.F


def weights(cfg, seed=3):
    from kv_cache_optimization_for_llm_amd.weights.random_init import random_state_dict
    state = random_state_dict(tensor_specs_for_config(cfg), seed, torch.bfloat16, 1.0)
    g = torch.Generator().manual_seed(seed)
    for name, t in state.items():
        if name.endswith((".b", ".sink", ".correction", ".lam", ".in", ".out", ".mix", "norm")):
            state[name] = (t.float() + torch.randn(t.shape, generator=g) * 0.3).to(torch.bfloat16)
    return plain.to_f64(state)


# ---------------------------------------------------------------- mechanisms
def test_softmax_with_a_sink_is_a_softmax_with_one_more_column_that_has_no_value():
    cfg = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 4, "scale": 0.7}
    g = torch.Generator().manual_seed(0)
    W = {f"p.{k}": torch.randn(s, generator=g, dtype=F) for k, s in
         dict(q=(16, 12), k=(8, 12), v=(4, 12), o=(12, 8)).items()}
    W.update({"p.q.norm": torch.ones(8, dtype=F), "p.k.norm": torch.ones(8, dtype=F), "p.sink": torch.tensor([0.3, -1.0], dtype=F)})
    h = torch.randn(9, 12, generator=g, dtype=F)
    got = plain.attention(h, W, "p.", cfg, 1e-6, window=4)
    q = plain.rms((h @ W["p.q"].T).view(9, 2, 8), 1e-6)
    k = plain.rms((h @ W["p.k"].T).view(9, 1, 8), 1e-6)
    v = (h @ W["p.v"].T).view(9, 1, 4)
    out = torch.zeros(9, 2, 4, dtype=F)
    for t in range(9):
        lo = max(0, t - 3)
        for head in range(2):
            s = torch.cat([(k[lo:t + 1, 0] @ q[t, head]) * 0.7, W["p.sink"][head:head + 1]])
            p = torch.softmax(s, 0)
            out[t, head] = p[:-1] @ v[lo:t + 1, 0]
    assert torch.allclose(got, out.reshape(9, 8) @ W["p.o"].T, atol=1e-12)


def test_rotation_as_complex_multiplication_and_linear_scaling_as_stretched_positions():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 2, 12, generator=g, dtype=F)
    pos = torch.tensor([0, 1, 2, 10, 11, 40])
    got = plain.rotate(x, pos, 8, 100.0)
    z = torch.complex(x[..., :4], x[..., 4:8])
    f = torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=F)
    r = z * torch.polar(torch.ones(6, 4, dtype=F), pos.to(F)[:, None] * f)[:, None, :]
    assert torch.allclose(got, torch.cat([r.real, r.imag, x[..., 8:]], -1), atol=1e-12)
    assert torch.allclose(plain.rotate(x, pos * 4, 8, 100.0, factor=4.0), got, atol=1e-12)


def test_matrix_memory_is_a_weighted_sum_over_earlier_tokens():
    """Without the running maximum: S_t = sum_j exp(i_j + sum_(l > j) f_l) k_j v_j^T, and the maximum cancels
    wherever |n . q| is the larger term of the denominator."""
    m = {"heads": 2, "dim": 4, "vdim": 3, "gate_cap": 5.0}
    g = torch.Generator().manual_seed(2)
    W = {f"p.{k}": torch.randn(s, generator=g, dtype=F) * 0.5 for k, s in
         dict(q=(8, 10), k=(8, 10), v=(6, 10), g=(6, 10), o=(10, 6), i=(2, 10), f=(2, 10)).items()}
    W.update({"p.i.b": torch.tensor([0.2, -0.4], dtype=F), "p.f.b": torch.tensor([1.0, 2.0], dtype=F),
              "p.norm": torch.ones(6, dtype=F)})
    h = torch.randn(7, 10, generator=g, dtype=F)
    got = plain.matrix_memory(h, W, "p.", m, 1e-5)
    q = (h @ W["p.q"].T).view(7, 2, 4) * 0.5
    k, v = (h @ W["p.k"].T).view(7, 2, 4), (h @ W["p.v"].T).view(7, 2, 3)
    gi = 5 * torch.tanh((h @ W["p.i"].T + W["p.i.b"]) / 5)
    gf = torch.nn.functional.logsigmoid(5 * torch.tanh((h @ W["p.f"].T + W["p.f.b"]) / 5))
    o = torch.zeros(7, 2, 3, dtype=F)
    for t in range(7):
        for hd in range(2):
            logw = torch.stack([gi[j, hd] + gf[j + 1:t + 1, hd].sum() for j in range(t + 1)])
            mx = torch.clamp(torch.cat([logw, gf[:t + 1, hd].sum()[None]]).max(), min=-math.inf)
            # the running maximum of the recurrence, by its own definition
            mrun = torch.tensor(0.0, dtype=F)
            for j in range(t + 1):
                mrun = torch.maximum(gf[j, hd] + mrun, gi[j, hd])
            w = torch.exp(logw - mrun)
            num = (w[:, None] * v[:t + 1, hd] * (k[:t + 1, hd] @ q[t, hd])[:, None]).sum(0)
            nq = (w * (k[:t + 1, hd] @ q[t, hd])).sum()
            o[t, hd] = num / (torch.maximum(nq.abs(), torch.exp(-mrun)) + 1e-6)
    o = plain.rms(o, 1e-5).reshape(7, 6) * torch.sigmoid(h @ W["p.g"].T)
    assert torch.allclose(got, o @ W["p.o"].T, atol=1e-10)


def test_real_gated_recurrence_in_closed_form_and_its_convolution_against_conv1d():
    m = {"width": 6, "blocks": 2, "conv": 3}
    g = torch.Generator().manual_seed(3)
    W = {f"p.{k}": torch.randn(s, generator=g, dtype=F) * 0.6 for k, s in
         dict(y=(6, 5), x=(6, 5), conv=(6, 3), ra=(2, 3, 3), ri=(2, 3, 3), o=(5, 6), lam=(6,)).items()}
    W.update({f"p.{k}": torch.randn(s, generator=g, dtype=F) * 0.3 for k, s in
              {"y.b": (6,), "x.b": (6,), "conv.b": (6,), "ra.b": (2, 3), "ri.b": (2, 3)}.items()})
    h = torch.randn(8, 5, generator=g, dtype=F)
    got = plain.rglru(h, W, "p.", m)
    x = (h @ W["p.x"].T + W["p.x.b"]).T[None]
    u = torch.nn.functional.conv1d(torch.nn.functional.pad(x, (2, 0)), W["p.conv"][:, None, :], W["p.conv.b"], groups=6)[0].T
    dense_a = torch.block_diag(*W["p.ra"])
    dense_i = torch.block_diag(*W["p.ri"])
    r = torch.sigmoid(u @ dense_a.T + W["p.ra.b"].reshape(-1))
    i = torch.sigmoid(u @ dense_i.T + W["p.ri.b"].reshape(-1))
    a = torch.exp(-8 * r * torch.nn.functional.softplus(W["p.lam"]))
    b = torch.sqrt(1 - a * a) * i * u
    S = torch.stack([sum(a[j + 1:t + 1].prod(0) * b[j] for j in range(t + 1)) for t in range(8)])
    y = plain.gelu_tanh(h @ W["p.y"].T + W["p.y.b"])
    assert torch.allclose(got, (S * y) @ W["p.o"].T, atol=1e-12)


def test_groups_hide_experts_behind_minus_infinity_and_weights_use_the_plain_scores():
    mlp = U.moe(6, 2, 4, 1.0, groups=(3, 1), scale=2.0)
    W = {"p.router": torch.zeros(6, 3, dtype=F), "p.correction": torch.tensor([-2.0, -2.1, -0.9, -3.0, -1.0, -1.0], dtype=F)}
    h = torch.zeros(1, 3, dtype=F)
    # scores are all 0.5: choice scores -1.5 -1.6 | -0.4 -2.5 | -0.5 -0.5; group sums -3.1, -2.9, -1.0: the last group wins,
    # though the single best expert (2) lies in another one
    idx, w, choice = plain.route(h, W, "p.", mlp)
    assert sorted(idx[0].tolist()) == [4, 5] and torch.isinf(choice[0, :4]).all()
    assert torch.allclose(w, torch.full((1, 2), 1.0, dtype=F))          # 0.5 / (0.5 + 0.5) * 2


def test_one_copy_of_the_stream_with_unit_weights_is_the_plain_residual_stream():
    cfg = copy.deepcopy(U.CFG_B)
    W = weights(cfg)
    toks = U.prompt(cfg, 12, 1)
    want = plain.forward(cfg, W, toks)
    cfg1 = dict(cfg, streams=1)
    W1 = dict(W)
    for i, layer in enumerate(cfg["layers"]):
        for q in (1, 2):
            W1[f"l{i}.hc{q}.in"] = W1[f"l{i}.hc{q}.out"] = torch.ones(1, dtype=F)
            W1[f"l{i}.hc{q}.mix"] = torch.ones(1, 1, dtype=F)
    assert torch.allclose(plain.forward(cfg1, W1, toks), want, atol=1e-10)


def test_the_model_is_causal_and_a_looped_run_is_the_same_layers_listed_again():
    cfg = copy.deepcopy(U.CFG_A)
    W = weights(cfg)
    toks = U.prompt(cfg, 30, 2)
    full = plain.forward(cfg, W, toks)
    assert torch.allclose(plain.forward(cfg, W, toks[:17]), full[:17], atol=1e-9)
    assert plain.run_order(cfg) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert plain.run_order({"layers": [0] * 3}) == [0, 1, 2]


# ---------------------------------------------------------------- the engine's description
def test_run_order_slots_and_tensor_names():
    config, spec = spec_for_config(U.CFG_A)
    assert [c.layer for c in spec.order] == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert [c.cache for c in spec.order] == list(range(9))            # every pass over slots of its own
    assert spec.streams == 3 and spec.residual_dtype == "float32"
    names = set(tensor_specs_for_config(U.CFG_A))
    for name in ("embed", "head", "final.norm", "final.norm.b", "l0.mix.conv.b", "l0.mix.ra", "l0.mlp.up", "l0.hc1.mix",
                 "l1.mix.q.norm", "l1.mix.sink", "l1.mlp.e5.gate", "l1.mlp.shared.sg", "l1.mlp.correction", "l1.hc2.in",
                 "l2.mix.left.k.norm", "l2.mix.right.i.b", "l2.mix.right.norm", "l3.norm1.b", "l4.mix.lam"):
        assert name in names, name
    assert "l3.norm2" not in names and "l3.hc2.in" not in names       # a layer without a feed-forward
    assert not any(".hc" in n for n in tensor_specs_for_config(U.CFG_B))          # no copies: no such tensors
    assert tensor_specs_for_config(U.CFG_C)["l0.hc1.mix"].shape == (1, 1)
    assert tensor_specs_for_config(U.CFG_A)["l2.mix.right.f"].shape == (3, 96)


def _broken(edit):
    cfg = copy.deepcopy(U.CFG_A)
    edit(cfg)
    return cfg


@pytest.mark.parametrize("edit", [
    lambda c: c.pop("vocab"),
    lambda c: c["norm"].pop("eps"),
    lambda c: c.update(streams=0),
    lambda c: c.update(streams=9),
    lambda c: c.update(loop={"start": 2, "stop": 2, "times": 2}),
    lambda c: c.update(loop={"start": 0, "stop": 6, "times": 1}),
    lambda c: c["layers"][0].update(type="lstm"),
    lambda c: c["layers"][0]["mixer"].update(blocks=5),
    lambda c: c["layers"][0]["mixer"].update(conv=18),
    lambda c: c["layers"][0]["mlp"].update(kind="gated"),
    lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][1]["mixer"].update(dim=30),
    lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34),
    lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7),
    lambda c: c["layers"][1]["mixer"]["mask"].update(size=0),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=7),
    lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4),
    lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=4),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=5),
    lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"),
    lambda c: c["layers"][2]["mixer"]["right"].update(gate_cap=0.0),
    lambda c: c["layers"][2]["mixer"].pop("left_scale"),
    lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].update(factor=0.0),
])
def test_configurations_that_cannot_run_are_refused(edit):
    with pytest.raises(ConfigError):
        spec_for_config(_broken(edit))
