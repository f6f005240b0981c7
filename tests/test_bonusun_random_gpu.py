"""Bonusun models drawn at random - layer order, loops, copies of the stream, widths, head counts and sizes,
rotation widths and scalings, windows, taps, runs of channels, routers with and without groups, constants,
missing feed-forwards - stepped through a random mixed schedule on a small pool and compared with the plain
implementation, in both number formats."""
import numpy as np
import pytest

import bonusun_util as U
import replay_util as R
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions

pytestmark = pytest.mark.gpu


def random_config(seed: int) -> dict:
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]      # noqa: E731
    width = pick(64, 72, 96, 100, 128, 160, 256)

    def mlp():
        r = rng.random()
        if r < 0.15:
            return None
        if r < 0.3:
            return U.dense(pick(48, 100, 256))
        experts, groups = pick((1, None), (2, None), (3, None), (4, (2, 1)), (6, (3, 2)), (8, (4, 2)), (8, (8, 3)), (12, (3, 2)),
                               (16, (2, 2)), (9, (3, 3)), (5, None))
        per = experts if groups is None else experts // groups[0] * groups[1]
        top = int(rng.integers(1, min(per, 6) + 1))
        return U.moe(experts, top, pick(16, 24, 32, 64, 96), pick(0.5, 1.0, 7.0), groups=groups, scale=pick(None, 1.0, 2.5),
                     shared=pick(None, (16, 1.0), (64, 2.0)))

    def attention():
        kv, dim = pick(1, 2, 3), pick(8, 16, 20, 32, 48, 64, 128)
        rot = pick(None, (dim, 10000.0), (dim // 4 * 2, 300000.0), (4, 50.0))
        return U.attention(kv * pick(1, 2, 4), kv, dim, pick(dim, 8, 16, 32, 80), pick(0.1, 0.125, 0.3), rot=rot,
                           window=pick(None, None, 1, 5, 16, 33, 80), factor=pick(None, 2.0, 8.0) if rot else None)

    layers = []
    for i in range(int(rng.integers(2, 6))):
        kind = pick("attention", "parallel", "rglru")
        if kind == "attention":
            layers.append(U.attention_layer(attention(), mlp()))
        elif kind == "parallel":
            right = (pick(1, 2, 4), pick(8, 16, 32, 40, 64, 136), pick(8, 24, 48, 64), float(pick(3.0, 5.0, 12.0)))
            layers.append(U.parallel_layer(attention(), right, pick(0.5, 1.0, 1.2), pick(0.5, 1.0, 1.7), mlp()))
        else:
            blocks = pick(1, 2, 4, 8)
            layers.append(U.rglru_layer(blocks * pick(8, 16, 24, 40, 80), blocks, pick(1, 2, 3, 4, 7), mlp()))
    cfg = {"architecture": "Bonusun", "vocab": pick(64, 101, 256, 333), "width": width, "norm": {"eps": pick(0.02, 0.05, 0.1)},
           "residual_mult": pick(0.5, 0.7, 1.0, 1.4), "layers": layers}
    streams = pick(None, 1, 2, 4, 5)
    if streams is not None:
        cfg["streams"] = streams
    if rng.random() < 0.5:
        a = int(rng.integers(0, len(layers)))
        cfg["loop"] = {"start": a, "stop": int(rng.integers(a + 1, len(layers) + 1)), "times": int(rng.integers(1, 4))}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(14))
def test_random_models_under_random_schedules(seed, dtype, tmp_path, gpu):
    cfg = random_config(3000 + seed)
    folder, state = U.write_model(str(tmp_path / "m"), cfg, seed, gain=0.8)
    rng = np.random.default_rng(seed)
    lengths = [int(n) for n in rng.integers(1, 140, size=7)]
    reqs = {f"q{i}": U.prompt(cfg, n, 13 * i + seed) for i, n in enumerate(lengths)}
    steps = R.mixed(reqs, seed=seed, max_live=4, chunk_sizes=(2, 3, 7, 16, 40))
    eng = Engine(folder, EngineOptions(dtype=dtype, page_size=16, cache_tokens=R.max_live_tokens(steps, unit=16),
                                       max_seqs=4, max_seq_len=160, max_batch_tokens=1024, use_graphs=False))
    rows, routes = U.run_steps(eng, steps, cfg)
    assert len(rows) == sum(lengths)
    # (in bfloat16 a router deep in a random model sees every earlier layer's rounding: its choice is held to
    # the rows' limits there; in 32-bit to the gap)
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs, routes, dtype, None if dtype == "float32" else 0.3), dtype,
                  f"model {cfg}")
    eng.cache.check()
    assert eng.cache.free_seats == 4 and all(g.free_pages() == g.num_pages for g in eng.cache.groups)
