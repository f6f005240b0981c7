"""The Bonusun decoder in the engine against the plain implementation (``plain_bonusun``).

Small configurations of their own (``bonusun_util``: other sizes, head counts, layer orders, loops,
windows, taps, routers and constants than any served model; also values that make two things equal, 1
or absent), seeded weights with spread-out scores.  Every schedule - whole prompts, token-by-token
decoding, portions down to two tokens, mixed batches on a pool so small that pages and seats come back -
must give the logits of the plain whole-sequence forward pass, in both number formats.  The plain experts
are run with the choices the engine's routers made; every choice that differs from the plain router's own
must be a close call there.
"""
import numpy as np
import pytest
import torch

import bonusun_util as U
import plain_bonusun as plain
import replay_util as R
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
from kv_cache_optimization_for_llm_amd.engine.runner import LLM, ServeOptions

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    base = tmp_path_factory.mktemp("bonusun")
    return {name: (cfg, *U.write_model(str(base / name), cfg, seed)) for name, (cfg, seed) in U.CONFIGS.items()}


def engine_for(folder, dtype, **kw):
    opts = dict(dtype=dtype, page_size=16, cache_tokens=1024, max_seqs=4, max_seq_len=512, max_batch_tokens=1024,
                use_graphs=False)
    opts.update(kw)
    return Engine(folder, EngineOptions(**opts))


REQUESTS = {"A": [1, 2, 9, 40, 77], "B": [3, 33, 70], "C": [1, 5, 47, 150], "D": [2, 35, 64], "E": [2, 44, 101]}


def requests_for(name, cfg):
    return {f"{name}{i}": U.prompt(cfg, n, 100 * i + n) for i, n in enumerate(REQUESTS[name])}


def check(eng, cfg, state, reqs, steps, dtype, what, close_call=None, tolerance=None):
    rows, routes = U.run_steps(eng, steps, cfg)
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs, routes, dtype, close_call), dtype, what, tolerance)
    eng.cache.check()
    return rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_whole_prompts_and_the_first_tokens(name, dtype, models, gpu):
    cfg, folder, state = models[name]
    reqs = requests_for(name, cfg)
    eng = engine_for(folder, dtype)
    rows = check(eng, cfg, state, reqs, R.whole(reqs), dtype, "whole")
    assert len(rows) == sum(len(t) for t in reqs.values())
    assert eng.cache.free_seats == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_prefill_against_token_by_token_decoding(name, dtype, models, gpu):
    """Most of a request in one step, the rest one token at a time (windows pass over decoded tokens; the
    states, the running maxima and the convolutions' last inputs are carried from step to step); and a
    request decoded from its very first token on."""
    cfg, folder, state = models[name]
    reqs = {k: v for k, v in requests_for(name, cfg).items() if len(v) > 30}
    eng = engine_for(folder, dtype)
    check(eng, cfg, state, reqs, R.tail_decoded(reqs, tail=45), dtype, "decode")
    first = {"solo": U.prompt(cfg, 60, 9)}
    check(eng, cfg, state, first, R.tail_decoded(first, tail=59), dtype, "decode from the first token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(2,), (7, 16, 5, 2, 33, 3, 64, 2), (17, 1, 1, 30)])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_portions_of_any_size(name, sizes, dtype, models, gpu):
    cfg, folder, state = models[name]
    reqs = {k: v for k, v in requests_for(name, cfg).items() if len(v) > 8}
    eng = engine_for(folder, dtype, page_size=8 if name == "A" else 16)
    check(eng, cfg, state, reqs, R.chunked(reqs, sizes), dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, seed", [("A", 0), ("B", 1), ("B", 2), ("C", 3), ("C", 4), ("D", 5), ("E", 6)])
def test_mixed_batches_on_a_small_pool_reuse_pages_and_seats(name, seed, dtype, models, gpu):
    cfg, folder, state = models[name]
    lengths = [40, 3, 90, 25, 61, 2, 130, 47, 33]
    reqs = {f"m{i}": U.prompt(cfg, n, 7 * i + seed) for i, n in enumerate(lengths)}
    steps = R.mixed(reqs, seed=seed, max_live=3)
    pool = R.max_live_tokens(steps, unit=16)
    eng = engine_for(folder, dtype, cache_tokens=pool, max_seqs=3, max_seq_len=192)
    rows = check(eng, cfg, state, reqs, steps, dtype, "mixed")
    assert len(rows) == sum(lengths)
    stats = eng.cache.stats()
    assert (stats["pages_reused"] > 0 or not eng.cache.groups) and stats["running"] == 0
    assert all(g.free_pages() == g.num_pages for g in eng.cache.groups)


def test_a_seat_that_is_taken_again_starts_from_an_empty_state(models, gpu):
    """One seat: every request inherits the seat, the pages and the state rows (matrices, normalisers,
    running maxima, recurrent states, convolution inputs) of the one before."""
    cfg, folder, state = models["A"]
    reqs = {f"s{i}": U.prompt(cfg, n, 40 + i) for i, n in enumerate([50, 7, 31, 2])}
    eng = engine_for(folder, "float32", max_seqs=1, cache_tokens=64, max_seq_len=64)
    check(eng, cfg, state, reqs, R.chunked(reqs, (9, 4)), "float32", "one seat")


def test_a_request_alone_and_in_a_batch_give_the_same_logits(models, gpu):
    """Logits of a (request, position) do not depend on the cut, the batch, the pages or the seat, beyond
    rounding (a recurrence's sums are formed in an order that follows the portion's length)."""
    cfg, folder, state = models["C"]
    reqs = {f"b{i}": U.prompt(cfg, n, 50 + i) for i, n in enumerate([70, 21, 44])}
    eng = engine_for(folder, "float32")
    alone = U.run_steps(eng, R.whole(reqs))
    together = U.run_steps(eng, R.mixed(reqs, seed=4, max_live=3, chunk_sizes=(2, 3, 16, 9)))
    assert alone.keys() == together.keys()
    for key in alone:
        assert U.row_error(together[key], alone[key]) <= 2e-5, str(key)


@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding_keeps_the_states_exact(name, models, gpu):
    """Four hundred single-token steps behind a short prompt, two requests beside each other."""
    cfg, folder, state = models[name]
    reqs = {"l0": U.prompt(cfg, 420, 1), "l1": U.prompt(cfg, 409, 2)}
    steps, n = [], 0
    steps.append({"step": n, "entries": [{"id": r, "tokens": t[:12], "want": [11]} for r, t in reqs.items()], "end": []})
    for i in range(12, 420):
        n += 1
        ent = [{"id": r, "tokens": t[i:i + 1], "want": [0]} for r, t in reqs.items() if i < len(t)]
        steps.append({"step": n, "entries": ent, "end": [r for r, t in reqs.items() if i == len(t) - 1]})
    eng = engine_for(folder, "float32")
    check(eng, cfg, state, reqs, steps, "float32", "long decoding")


def _sharp(cfg, gain):
    """Queries and keys of every attention scaled up (through their norms' weights), so that the softmax is
    sharp: one key - or the sink - carries nearly all the weight, and a key wrongly seen or wrongly hidden,
    or a sink left out, moves the row by far more than rounding."""
    def edit(state):
        for i, layer in enumerate(cfg["layers"]):
            for p in {"attention": [f"l{i}.mix."], "parallel": [f"l{i}.mix.left."]}.get(layer["type"], []):
                for key in ("q.norm", "k.norm"):
                    state[p + key] = (state[p + key].float() * gain).to(torch.bfloat16)
                state[p + "sink"] = (state[p + "sink"].float() * 3.0 + 2.0).to(torch.bfloat16)
    return edit


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, gain, cuts", [("A", 4.0, (24, 23, 2, 7, 6, 8, 48, 1, 21)),
                                              ("C", 2.0, (32, 31, 2, 16, 15, 18, 100, 1, 47, 96))])
def test_sharp_scores_at_window_edges_sinks_and_far_keys(name, gain, cuts, dtype, tmp_path, gpu):
    """With sharp softmaxes every row depends on WHICH keys it sees and on the sink: the positions just inside
    and just outside every window, in prompts, in portions that end and start at a window's length and one
    token off it, and decoded one by one; and - in the layers without a window - a key hundreds of positions
    back.  (A: the kernels for values of another size than the keys; C: the bf16 engine's matrix-core kernels.)"""
    cfg = U.CONFIGS[name][0]
    if dtype == "bfloat16":
        gain = min(gain, 2.0)          # (in 16 bits a softmax four times as sharp turns rounding into other keys)
    if name == "A":
        # (every run of a layer with softmaxes that sharp doubles or triples what rounding did before it: the
        # looped layers run once here, five layer runs in all)
        cfg = dict(cfg, loop=dict(cfg["loop"], times=1))
    folder, state = U.write_model(str(tmp_path / "sharp"), cfg, 21, edit=_sharp(cfg, gain))
    reqs = {"e0": U.prompt(cfg, 75, 1), "e1": U.prompt(cfg, 340, 2)}
    eng = engine_for(folder, dtype)
    # (softmaxes that sharp multiply the rounding of what they read: a 32-bit row may be off by 1e-3 - a key
    # wrongly seen or hidden moves it by a hundred times that - and in bfloat16 the routers behind them see it:
    # there a router's choice is held to the rows' limits alone in A and to gaps of 0.3 in C; in 32-bit no gap
    # is forgiven)
    close = None if dtype == "float32" else (1.0 if name == "A" else 0.3)
    tol = 1e-3
    check(eng, cfg, state, reqs, R.whole(reqs), dtype, "whole", close, tol)
    check(eng, cfg, state, reqs, R.chunked(reqs, cuts), dtype, "cuts at window lengths", close, tol)
    check(eng, cfg, state, {"e0": reqs["e0"]}, R.tail_decoded({"e0": reqs["e0"]}, tail=60), dtype, "decoded over window edges", close, tol)
    check(eng, cfg, state, {"e1": reqs["e1"]}, R.tail_decoded({"e1": reqs["e1"]}, tail=20), dtype, "decoded far from the start", close, tol)
    side = {f"s{i}": U.prompt(cfg, n, 30 + i) for i, n in enumerate([40, 65, 110, 129])}
    check(eng, cfg, state, side, R.mixed(side, seed=2, max_live=4, chunk_sizes=(31, 33, 17)), dtype, "decoded side by side", close, tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_trace_runner_replays_a_mixed_schedule(dtype, models, tmp_path, gpu):
    """``bin/trace_run`` (graphs and all) on a mixed schedule; fp32 against the plain model, bf16 against the
    eager engine (which the other tests hold against the plain model with its own routes)."""
    cfg, folder, state = models["C"]
    reqs = {f"t{i}": U.prompt(cfg, n, 11 + i) for i, n in enumerate([30, 2, 75, 18, 52])}
    steps = R.mixed(reqs, seed=5, max_live=4)
    rows = R.run_trace(folder, dtype, steps, R.max_live_tokens(steps), str(tmp_path / "out"), cfg["vocab"])
    assert R.cache_stats(str(tmp_path / "out"))["pages_reused"] > 0
    eng = engine_for(folder, dtype, cache_tokens=R.max_live_tokens(steps), max_seqs=4)
    eager, routes = U.run_steps(eng, steps, cfg)
    U.assert_rows(eager, U.expected_rows(cfg, state, reqs, routes, dtype), dtype, "eager")
    for key in eager:
        e = U.row_error(rows[key], eager[key])
        assert e <= (2e-5 if dtype == "float32" else 3e-2), f"{key}: the runner is off the engine by {e:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(name, dtype, models, gpu):
    cfg, folder, state = models[name]
    W = plain.to_f64(state)
    prompts = [U.prompt(cfg, n, 3 + n) for n in (1, 12, 37, 64, 5, 90)]
    llm = LLM(folder, EngineOptions(dtype=dtype, max_seqs=3, max_seq_len=160, cache_tokens=480),
              ServeOptions(chunk_size=16, max_batch_tokens=48))
    got, reasons = llm.generate(prompts, max_new_tokens=24, ignore_eos=True, return_reasons=True)
    assert reasons == ["length"] * len(prompts)
    good = total = 0
    for p, g in zip(prompts, got):
        assert len(g) == 24
        logits = plain.forward(cfg, W, list(p) + list(g)).numpy()
        for i, tok in enumerate(g):
            row = logits[len(p) + i - 1]
            slack = (1e-3 if dtype == "float32" else 6e-2) * (row.max() - row.mean())
            good += row[tok] >= row.max() - slack
            total += 1
    # (a router's close call that falls the other way moves a row by more than rounding: a few picks may differ)
    assert good >= (total if dtype == "float32" else 0.8 * total), f"{total - good} of {total} picks are not the best"
    llm.engine.cache.check()
    assert llm.engine.cache.free_seats == 3


@pytest.mark.parametrize("name", ["A", "C", "E"])
def test_decode_steps_from_graphs_equal_eager_steps(name, models, gpu):
    """A bf16 decode step replayed from its HIP graph gives bit for bit what the eager step gives (the copies
    of the stream, states, convolution inputs and routed experts included), replay after replay."""
    cfg, folder, state = models[name]
    reqs = {f"g{i}": U.prompt(cfg, n, 31 + i) for i, n in enumerate([48, 80])}
    steps = R.tail_decoded(reqs, tail=20)
    eager = U.run_steps(engine_for(folder, "bfloat16"), steps)
    eng = engine_for(folder, "bfloat16", use_graphs=True)
    assert eng.graphs is not None
    replayed = U.run_steps(eng, steps)
    assert eng.graphs.replays > 0
    for key in eager:
        np.testing.assert_array_equal(eager[key], replayed[key], err_msg=str(key))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_contiguous_cache_mode_gives_the_logits_of_the_plain_model(dtype, models, gpu):
    cfg, folder, state = models["C"]
    reqs = {f"c{i}": U.prompt(cfg, n, 90 + i) for i, n in enumerate([70, 33, 121])}
    eng = engine_for(folder, dtype, cache_mode="contiguous", cache_tokens=4 * 128, max_seq_len=128)
    check(eng, cfg, state, reqs, R.mixed(reqs, seed=9, max_live=3), dtype, "contiguous")


def test_the_serving_process_serves_the_model(models, tmp_path, gpu):
    """``cli.client`` starts ``cli.serve`` on the model folder: every sequence emits its budget (scheduler,
    sampler and command line are the ones every architecture uses)."""
    import json
    import os
    import subprocess
    import sys
    cfg, folder, state = models["A"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "paged.json"
    env = dict(os.environ, IGNORE_EOS="1", ORCA_POLICY="oracle", PYTHONPATH=root)
    cmd = [sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.client", folder, "5", "--prompt-len", "37",
           "--max-new-tokens", "10", "--num-seqs", "2", "--out", str(out), "--", "--dtype", "float32",
           "--cache-mode", "paged", "--max-seqs", "4", "--max-seq-len", "64", "--cache-tokens", "384",
           "--chunk-size", "8", "--max-batch-tokens", "24"]
    proc = subprocess.run(cmd, env=env, cwd=root, capture_output=True, text=True, timeout=280)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    r = json.load(open(out))
    assert r["status"] == "ok" and r["sequences_done"] == 10 and r["tokens"] == 100
    assert r["count_mismatches"] == 0 and r["budget_mismatches"] == 0 and r["errors"] == []


def test_the_sweep_command_runs_a_configuration_file_of_this_architecture(models, tmp_path, gpu):
    import json
    import os
    from kv_cache_optimization_for_llm_amd.cli import sweep
    cfg, folder, state = models["C"]
    out = tmp_path / "sweep.jsonl"
    assert sweep.main(["--shapes", os.path.join(folder, "config.json"), "--batches", "3", "--cache-modes", "paged",
                       "--prompt-len", "40", "--prompt-min", "5", "--workload", "mixed", "--new-tokens", "9",
                       "--max-seqs", "2", "--out", str(out)]) == 0
    line, = [json.loads(l) for l in out.read_text().splitlines()]
    assert line["requests_done"] == 3 and line["tokens_emitted"] == 27 and line["finish_reasons"] == {"length": 3}
    assert line["pages_reused"] > 0
