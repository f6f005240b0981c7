#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.2-1B shape, random bf16 weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is decoded tokens per second of the default run: a batch of 8
requests whose contexts end at 8,192 tokens, driven by the serving loop; a "step" is one decode
step (scheduling, model forward over the paged cache, greedy sampling, token ids back on the host).
The same line carries the 2,048-token prefill; the decode roofline (bytes the step has to read /
time / HBM peak, and against what a plain read stream gets from this GPU); ``points``: batch 1 and
batch 64 at the same context and batches 1, 8 and 64 with 512-token prompts and 256 generated
tokens, each with its step time, bytes and fraction of the HBM peak, and the serving loop at the
3B and 8B layer sizes (mixed prompt lengths; paged against contiguous cache occupancy).
``points`` also holds the device time per class of kernel of one decode step and of the prefill
(``kclass_...``; ``--no-kernel-classes`` leaves them out) and, for the serving runs, pages reused,
preemptions and fragmentation failures.

    python bench.py --design gadopel|radilix|lomodra|bonusun [--layers 8]

is another measurement with a JSON line of its own (the default run above is untouched): prefill
and decode throughput of a Gadopel model at layer sizes of a served model (random weights), beside
a Llama model of equal width, depth, feed-forward and vocabulary, with the device time per class
of kernel of one decode step and one prefill of each.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# the benchmark configuration: Llama 3.2 1B shape
CONFIG_1B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048,
    intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
    head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16",
)
CONTEXT = 8192
PAGE = 16
PREFILL_TOKENS = 2048


def weight_bytes(cfg, elem=2):
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (q + 2 * kv) * H + H * q + 3 * I * H + 2 * H
    head = V * H if cfg["tie_word_embeddings"] else V * H      # the output matrix is read once either way
    return (L * per_layer + H + head) * elem


def kv_bytes_per_token(cfg, elem=2):
    return 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * elem


def prefill_flops(cfg, T):
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    linear = 2 * T * L * ((q + 2 * kv) * H + H * q + 3 * I * H)
    attn = L * 4 * cfg["num_attention_heads"] * cfg["head_dim"] * T * (T + 1) / 2
    return linear + attn + 2 * V * H


# --design gadopel: layers of width 2,048 with a feed-forward of 8,192.  Latent layers with 16
# heads of 128 + 64 query/key elements over rows of 512 + 64, windowed layers with 32 heads of 64
# over 8 kv heads and a window of 1,024 that keeps 64 first positions, in turn; the Llama beside it
# has 32 heads of 64 over 8 kv heads in every layer.
def gadopel_config(layers: int, vocab: int) -> dict:
    latent = {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 8192},
              "mixer": {"heads": 16, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "scale": 192 ** -0.5,
                        "rot": {"base": 10000.0, "dims": 64}}}
    windowed = {"type": "attention", "mlp": {"kind": "dense", "ff": 8192},
                "mixer": {"heads": 32, "kv_heads": 8, "dim": 64, "vdim": 64, "scale": 1.0,
                          "mask": {"size": 1024, "keep_first": 64},
                          "rot": {"base": 500000.0, "dims": 64,
                                  "scaling": {"factor": 16.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}}
    return {"architecture": "Gadopel", "vocab": vocab, "width": 2048, "norm": {"eps": 1e-6},
            "layers": [latent if i % 2 == 0 else windowed for i in range(layers)], "max_positions": 8192}


# --design radilix: layers of width 2,048.  Three in four are mixers side by side - attention with
# 32 heads of 64 over 8 kv heads (rotation of half a head, biases, sigmoid gate) beside a gated delta
# rule with 8 value heads of 128 over 4 query/key heads of 128 and four taps -, every fourth is gated
# linear attention with 16 heads of 64 x 128; every layer has 16 routed experts of width 1,024 and 2
# identity experts, 4 choices a token (67 M expert weights a layer against the Llama layer's 50 M of
# feed-forward; a token uses a quarter of them).
# At another --width W the head counts and the experts' width scale with it (W / 64 attention heads over
# W / 256 kv heads, W / 256 delta-rule heads, W / 128 heads of gated linear attention, experts of W / 2).
def radilix_config(layers: int, vocab: int, width: int = 2048) -> dict:
    W = width
    mlp = {"kind": "moe", "expert": {"ff": W // 2}, "router": {"experts": 16, "identity": 2, "top": 4}}
    side = {"type": "parallel", "mlp": mlp, "mixer": {
        "left": {"heads": W // 64, "kv_heads": W // 256, "dim": 64, "vdim": 64, "scale": 0.125,
                 "rot": {"base": 500000.0, "dims": 32}},
        "right": {"heads": W // 256, "kv_heads": W // 512, "dim": 128, "vdim": 128, "conv": 4},
        "left_scale": 1.0, "right_scale": 0.5}}
    gla = {"type": "gla", "mlp": mlp, "mixer": {"heads": W // 128, "dim": 64, "vdim": 128, "tau": 16.0, "decay_rank": 16}}
    return {"architecture": "Radilix", "vocab": vocab, "width": W, "norm": {"eps": 1e-6}, "residual_mult": 0.7,
            "layers": [gla if i % 4 == 3 else side for i in range(layers)], "max_positions": 8192}


# --design lomodra: layers of width W in runs of four - softmax attention inside chunks of 1,024 positions
# (W / 64 heads of 64 over W / 256 kv heads, normed queries and keys), a delta rule with a decay per key
# channel (W / 256 value heads of 128 over W / 512 query/key heads of 128, four taps, ranks of 64), lightning
# attention (W / 128 heads of 64 x 128), and an attention layer that reads the first one's keys and values.
# Every layer has 16 gated experts of width 3 W / 8 (three matrices: 1.125 W^2 weights an expert, against
# the Radilix expert's W^2), 4 choices a token, one more expert of that width that every token uses, and a
# token input of 64 columns.  Beside it run the closest design, Radilix (recurrences and routed experts
# too), and the Llama model, both at the same width.
def lomodra_config(layers: int, vocab: int, width: int = 2048) -> dict:
    W = width
    mlp = {"kind": "moe", "expert": {"ff": 3 * W // 8}, "router": {"experts": 16, "top": 4}, "shared": {"ff": 3 * W // 8}}
    attn = {"heads": W // 64, "kv_heads": W // 256, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 1024}}
    kinds = [
        lambda i: {"type": "attention", "mlp": mlp, "mixer": dict(attn)},
        lambda i: {"type": "channel_delta", "mlp": mlp, "mixer": {"heads": W // 256, "kv_heads": W // 512, "dim": 128,
                                                                   "vdim": 128, "conv": 4, "decay_rank": 64, "gate_rank": 64}},
        lambda i: {"type": "lightning", "mlp": mlp, "mixer": {"heads": W // 128, "dim": 64, "vdim": 128,
                                                               "decay": [1.0 - 2.0 ** -(3 + 5 * h / max(1, W // 128 - 1))
                                                                         for h in range(W // 128)]}},
        lambda i: {"type": "attention", "mlp": mlp, "mixer": dict(attn, kv_from=i - 3)},
    ]
    return {"architecture": "Lomodra", "vocab": vocab, "width": W, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
            "token_side": {"dim": 64}, "layers": [kinds[i % 4](i) for i in range(layers)], "max_positions": 8192}


# --design bonusun: layers of width W in runs of four over four copies of the stream - a real-gated linear
# recurrent unit (W channels in runs of 256, four taps), softmax attention inside a window of 1,024 positions
# (W / 64 heads of 64 over W / 256 kv heads, normed queries and keys, a sink), such an attention without a
# window beside a matrix memory (W / 128 heads of 64 x 128), and windowed attention again.  Every layer has 16
# clamped gated experts of width 3 W / 8 in 4 groups of which 2 are kept, 4 choices a token, and one more
# expert of that width that every token uses.  Beside it run the closest design, Radilix (mixers side by side,
# recurrences and routed experts too), and the Llama model, both at the same width.
def bonusun_config(layers: int, vocab: int, width: int = 2048) -> dict:
    W = width
    mlp = {"kind": "moe", "expert": {"ff": 3 * W // 8, "limit": 7.0},
           "router": {"experts": 16, "top": 4, "groups": {"count": 4, "keep": 2}, "scale": 2.5},
           "shared": {"ff": 3 * W // 8, "limit": 7.0}}
    attn = {"heads": W // 64, "kv_heads": W // 256, "dim": 64, "vdim": 64, "scale": 0.125, "rot": {"base": 500000.0, "dims": 64}}
    kinds = [
        {"type": "rglru", "mlp": mlp, "mixer": {"width": W, "blocks": W // 256, "conv": 4}},
        {"type": "attention", "mlp": mlp, "mixer": dict(attn, mask={"size": 1024})},
        {"type": "parallel", "mlp": mlp, "mixer": {"left": dict(attn), "left_scale": 1.0, "right_scale": 0.5,
                                                   "right": {"heads": W // 128, "dim": 64, "vdim": 128, "gate_cap": 12.0}}},
        {"type": "attention", "mlp": mlp, "mixer": dict(attn, mask={"size": 1024})},
    ]
    return {"architecture": "Bonusun", "vocab": vocab, "width": W, "norm": {"eps": 1e-6}, "residual_mult": 0.7, "streams": 4,
            "layers": [kinds[i % 4] for i in range(layers)], "max_positions": 8192}


def design_comparison(args) -> int:
    import torch
    from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
    from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
    from kv_cache_optimization_for_llm_amd.ops import kernels as K

    layers, vocab = args.layers or 8, 32000
    llama = dict(CONFIG_1B, num_hidden_layers=layers, vocab_size=vocab, tie_word_embeddings=False)
    design, width = args.design, args.width
    if width != 2048:
        if design not in ("radilix", "lomodra", "bonusun") or width % 512 or not 512 <= width <= 8192:
            print("--width: a multiple of 512 from 512 to 8192, for --design radilix, lomodra or bonusun")
            return 2
        llama.update(hidden_size=width, intermediate_size=4 * width, num_attention_heads=width // 64,
                     num_key_value_heads=width // 256)
    if design == "lomodra":
        configs = {design: lomodra_config(layers, vocab, width), "radilix": radilix_config(layers, vocab, width), "llama": llama}
    elif design == "bonusun":
        configs = {design: bonusun_config(layers, vocab, width), "radilix": radilix_config(layers, vocab, width), "llama": llama}
    elif design == "radilix":
        configs = {design: radilix_config(layers, vocab, width), "llama": llama}
    else:
        configs = {design: gadopel_config(layers, vocab), "llama": llama}
    shapes = [(8, 4096), (32, 2048)]            # (requests, context) of the decode runs
    gen = torch.Generator().manual_seed(0)
    out = {}
    for name, cfg in configs.items():
        pool = max(b * (c + 2 * PAGE) for b, c in shapes)
        engine = Engine(None, EngineOptions(dtype="bfloat16", page_size=PAGE, cache_tokens=pool, max_seqs=32,
                                            max_seq_len=8192, max_batch_tokens=8192, max_logit_rows=64),
                        config_dict=cfg, random_seed=0)
        stacked = [w for b in engine.model.blocks for w in (getattr(b.feed_forward, "w_up", None),
                                                            getattr(b.feed_forward, "w_down", None)) if w is not None]
        res = {"weight_gb": round(sum(t.numel() * t.element_size() for t in
                                      [lin.weight for lin in engine.model.linears()] + stacked) / 1e9, 3),
               "cache_bytes_per_token": engine.cache.page_bytes() // PAGE}

        def timed_prefill(tokens):
            prompt = [int(t) for t in torch.randint(0, vocab, (tokens,), generator=gen)]
            best = 1e9
            for i in range(5):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                engine.step([StepEntry(f"p{i}", prompt, [tokens - 1])])
                torch.cuda.synchronize()
                best = min(best, time.perf_counter() - t0) if i else best
                engine.release(f"p{i}")
            return best

        for tokens in (PREFILL_TOKENS,):
            sec = timed_prefill(tokens)
            res[f"prefill_{tokens}_tok_s"] = round(tokens / sec, 1)
            res[f"prefill_{tokens}_ms"] = round(sec * 1e3, 3)
        for batch, context in shapes:
            ids = [f"d{i}" for i in range(batch)]
            base = [int(t) for t in torch.randint(0, vocab, (context - args.steps - args.warmup - 4,), generator=gen)]
            for rid in ids:
                for lo in range(0, len(base), 4096):
                    engine.step([StepEntry(rid, base[lo:lo + 4096], [])])
            step = [StepEntry(rid, [7], [0]) for rid in ids]
            for _ in range(args.warmup + 2):
                engine.step(step)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                engine.step(step)
            torch.cuda.synchronize()
            sec = time.perf_counter() - t0
            res[f"decode_b{batch}_c{context}_tok_s"] = round(batch * args.steps / sec, 1)
            res[f"decode_b{batch}_c{context}_ms"] = round(sec / args.steps * 1e3, 4)
            if (batch, context) == shapes[0]:
                graphs, portion_graphs = engine.graphs, engine.portion_graphs
                engine.graphs = engine.portion_graphs = None        # launched one by one, events between
                engine.step(step)
                with K.KernelClassTimer() as timer:
                    engine.step(step)
                res[f"kclass_decode_b{batch}_c{context}_ms"] = timer.milliseconds()
                engine.graphs, engine.portion_graphs = graphs, portion_graphs
            for rid in ids:
                engine.release(rid)
        graphs, portion_graphs = engine.graphs, engine.portion_graphs
        engine.graphs = engine.portion_graphs = None
        prompt = [int(t) for t in torch.randint(0, vocab, (PREFILL_TOKENS,), generator=gen)]
        engine.step([StepEntry("kp0", prompt, [PREFILL_TOKENS - 1])])
        engine.release("kp0")
        with K.KernelClassTimer() as timer:
            engine.step([StepEntry("kp1", prompt, [PREFILL_TOKENS - 1])])
        res[f"kclass_prefill_{PREFILL_TOKENS}_ms"] = timer.milliseconds()
        engine.release("kp1")
        out[name] = res
        del engine
        import gc
        gc.collect()
        torch.cuda.empty_cache()
    b, c = shapes[0]
    print(json.dumps({"metric": f"{design}_decode_tokens_per_second", "value": out[design][f"decode_b{b}_c{c}_tok_s"],
                      "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                      "higher_is_better": True, "dtype": "bf16", "data": "synthetic (random weights, seeded token ids)",
                      "config": {"design": f"{design} beside " + " and ".join(n for n in configs if n != design), "layers": layers, "width": width, "ff": 4 * width,
                                 "vocab": vocab, "decode_shapes": shapes, "prefill_tokens": PREFILL_TOKENS},
                      "designs": out}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--design", choices=["gadopel", "radilix", "lomodra", "bonusun"], default=None,
                    help="another measurement (its own JSON line): a model of this design at the layer sizes of a "
                         "served model beside a Llama model of equal size; the default run is left as it is")
    ap.add_argument("--width", type=int, default=2048, help="--design radilix, lomodra or bonusun: the models' width (head counts and "
                    "feed-forward sizes scale with it)")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=CONTEXT)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the 16 of the configuration")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="leave the vendor GEMM library its own choice of algorithm (no timing at start-up)")
    ap.add_argument("--skip-points", action="store_true", help="only the default decode run and the prefill")
    ap.add_argument("--skip-large", action="store_true",
                    help="leave out the serving runs at the 3B and 8B layer sizes (about a minute together)")
    ap.add_argument("--no-kernel-classes", dest="kernel_classes", action="store_false",
                    help="leave out the device time per class of kernel (one decode step and the prefill with events "
                         "around every launch, launched one by one instead of replayed from graphs: a second or two)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2
    if args.design:
        return design_comparison(args)

    import torch
    from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
    from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner, ServeOptions

    cfg = dict(CONFIG_1B)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    max_batch = 64 if not args.skip_points else args.batch
    ctx = args.context
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], ctx)      # a longer --context
    # room for max_batch requests at the context, one more page each for the tokens decoded
    pool = max(max_batch * (ctx + 2 * PAGE), PREFILL_TOKENS + PAGE)      # and room for the prefill's prompt
    # the vendor library's algorithms are timed once, at start-up, for the row counts whose
    # products go to it here: the prefill's 2,048 tokens and decode batches above 16
    tune_rows = [] if args.no_gemm_tuning else [PREFILL_TOKENS] + [b for b in {args.batch, max_batch} if b > 16]
    engine = Engine(None, EngineOptions(dtype="bfloat16", page_size=PAGE, cache_tokens=pool,
                                        max_seqs=max_batch, max_seq_len=cfg["max_position_embeddings"],
                                        max_batch_tokens=32768, max_logit_rows=max(64, args.batch),
                                        gemm_tune_rows=tune_rows),
                    config_dict=cfg, random_seed=0)
    dev = engine.device
    gen = torch.Generator().manual_seed(0)

    def decode_run(batch, steps, warmup, context, decoded_before=0):
        """Times ``steps`` decode steps of ``batch`` requests through the serving loop (scheduler,
        step function, sampler; a step is launched while the host still waits for the previous
        step's tokens).  The prompts are prefilled first, in portions; their lengths are set so
        that the longest context ENDS at ``context``.  ``decoded_before``: the requests have been
        decoding for that many steps when the warm-up steps begin.  Returns (seconds, mean
        context length over the timed steps)."""
        budget = 32768
        runner = Runner(engine, ServeOptions(ignore_eos=True, run_ahead=True, max_batch_tokens=budget))
        warmup += decoded_before
        lead = warmup + steps + 2
        first = context - lead
        first -= (batch * first + budget - 1) // budget + 1      # steps that other requests' prompts take
        if first < 1:
            raise SystemExit(f"context {context} is too short for {steps} + {warmup} steps")
        for _ in range(batch):
            prompt = [int(t) for t in torch.randint(0, engine.vocab_size, (first,), generator=gen)]
            runner.submit(prompt, context - first - 1)
        sched = runner.scheduler
        while sched.waiting or any(s.prefilling for s in sched.running):
            runner.step()
        for _ in range(warmup):
            runner.step()
        torch.cuda.synchronize()
        if len(sched.running) != batch or any(s.prefilling for s in sched.running):
            raise SystemExit(f"bench: {len(sched.running)} of {batch} requests are decoding after the prompts "
                             f"(waiting {len(sched.waiting)}, preemptions {sched.preemptions}): the pool or the "
                             f"token budget does not fit context {context}")
        ctx0 = sum(s.computed for s in sched.running) / batch
        t0 = time.perf_counter()
        for _ in range(steps):
            runner.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(sched.running) == batch and max(s.computed for s in sched.running) <= context
        mean_ctx = ctx0 + steps / 2
        # drop the requests (their remaining budget is not part of the measurement)
        for rid in runner.live_requests():
            runner.cancel(rid)
        assert runner.idle()
        return dt, mean_ctx

    dt, mean_ctx = decode_run(args.batch, args.steps, args.warmup, ctx)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes(cfg) + args.batch * mean_ctx * kv_bytes_per_token(cfg)
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9

    # prefill of 2,048 tokens: one request, one step, logits at the last place
    prompt = [int(t) for t in torch.randint(0, engine.vocab_size, (PREFILL_TOKENS,), generator=gen)]
    pre_ms = []
    for i in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(f"p{i}", prompt, [PREFILL_TOKENS - 1])])
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t0) * 1e3)
        engine.release(f"p{i}")
    p_ms = min(pre_ms[1:])
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / (p_ms * 1e-3), 1), "tokens": PREFILL_TOKENS,
               "ms": round(p_ms, 3), "frac": round(flops / (p_ms * 1e-3) / (PEAK_TFLOPS["bf16"] * 1e12), 4)}

    points = {}

    def add_point(name, batch, steps, seconds, mean_context):
        """tok/s under the name itself; beside it the step's time, the bytes it has to read (every
        weight once, the cache of the live requests) and the fraction of the HBM peak that is."""
        ms = seconds / steps * 1e3
        gb = (weight_bytes(cfg) + batch * mean_context * kv_bytes_per_token(cfg)) / 1e9
        points[name] = round(batch * steps / seconds, 1)
        points[name + "_ms"] = round(ms, 4)
        points[name + "_gb"] = round(gb, 3)
        points[name + "_frac"] = round(gb / (ms * 1e-3) / HBM_PEAK_GBS, 4)

    if not args.skip_points:
        for b in (1, 64):
            k = max(16, args.steps // 2)
            d, c = decode_run(b, k, 8, ctx)
            add_point(f"decode_b{b}", b, k, d, c)
        # The default run again, with the requests 320 steps into their decoding when the same warm-up
        # and the same timed steps begin.  After a prefill (seconds of matrix products that ask
        # little of the memory) the first third of a second of decode steps runs 6-7 % slower than
        # all that follow: every kernel that streams weights takes 0.5-1 us longer, until the
        # memory has been busy for that long (one run of 8 x 8,192, 40 steps at a time: 1.227 ms
        # seven times, then 1.169, 1.150, 1.149 ..; kernel by kernel in a trace: down and output
        # 8.9 -> 7.9 us, gate/up 14.1 -> 13.1, Q/K/V 7.9 -> 7.4, attention 25.4 -> 24.8).  A server
        # that decodes is past that point; the default run, timed right after its prompts, is not.
        # Every point has such a twin, "..._sustained": about 0.4 s of decode steps first, or, where
        # the context has no room for them, the same run repeated until as much lies behind.
        if ctx >= 400 + args.warmup + args.steps + 64:
            d, c = decode_run(args.batch, args.steps, args.warmup, ctx, decoded_before=320)
            add_point(f"decode_b{args.batch}_sustained", args.batch, args.steps, d, c)
            for b, before in ((1, 400), (64, 96)):
                k = max(16, args.steps // 2)
                d, c = decode_run(b, k, 8, ctx, decoded_before=before)
                add_point(f"decode_b{b}_sustained", b, k, d, c)
        # the serving workload of the comparison: 512-token prompts, 256 generated tokens
        for b in (1, 8, 64):
            d, c = decode_run(b, 240, 8, 512 + 256)
            add_point(f"decode_b{b}_p512_g256", b, 240, d, c)
            spent = d
            while spent < 0.45:                  # the same run again until 0.45 s of decode steps lie behind
                d, c = decode_run(b, 240, 8, 512 + 256)
                spent += d
            d, c = decode_run(b, 240, 8, 512 + 256)
            add_point(f"decode_b{b}_p512_g256_sustained", b, 240, d, c)

    # what a plain read stream gets from this GPU's memory (the published peak is 8 TB/s)
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    probed_gbs = K.probe_read_bandwidth(dev)

    kernel_ms = None
    if args.kernel_classes:
        graphs, portion_graphs = engine.graphs, engine.portion_graphs
        engine.graphs = engine.portion_graphs = None           # launched one by one, so that events fit between
        kernel_ms = {}
        try:
            # eight requests decoding at the context's end
            ids = [f"k{i}" for i in range(args.batch)]
            base = [int(t) for t in torch.randint(0, engine.vocab_size, (ctx - 8,), generator=gen)]
            for rid in ids:
                for lo in range(0, len(base), 4096):
                    engine.step([StepEntry(rid, base[lo:lo + 4096], [])])
            step = [StepEntry(rid, [5], [0]) for rid in ids]
            engine.step(step)
            with K.KernelClassTimer() as timer:
                engine.step(step)
            kernel_ms[f"decode_b{args.batch}_eager"] = timer.milliseconds()
            for rid in ids:
                engine.release(rid)
            engine.step([StepEntry("kp0", prompt, [PREFILL_TOKENS - 1])])
            engine.release("kp0")
            with K.KernelClassTimer() as timer:
                engine.step([StepEntry("kp1", prompt, [PREFILL_TOKENS - 1])])
            kernel_ms[f"prefill_{PREFILL_TOKENS}_eager"] = timer.milliseconds()
            engine.release("kp1")
        finally:
            engine.graphs, engine.portion_graphs = graphs, portion_graphs

    # The serving loop at the layer sizes of the larger configurations (random weights, seeded
    # uniform token ids): 32 requests with prompts of 128 to 4,096 tokens and 128 new tokens each,
    # portions of 512, at the 3B sizes; 64 concurrent requests of 8,192 + 512 tokens at the 8B
    # sizes, once over the paged cache and once over the contiguous one (what is reserved against
    # what holds a token is the comparison the reference's paper makes).
    if not args.skip_large:
        import gc
        from kv_cache_optimization_for_llm_amd.cli import sweep
        del engine
        gc.collect()
        torch.cuda.empty_cache()
        mixed = sweep.build_parser().parse_args(
            ["--workload", "mixed", "--prompt-len", "4096", "--prompt-min", "128", "--new-tokens", "128",
             "--chunk-size", "512", "--max-batch-tokens", "4096", "--tune-gemm"])
        r = sweep.run_one(mixed, "3b", 32, "paged")
        points.update({"serve_3b_mixed_b32_tok_s": round(r["tokens_emitted"] / r["wall_s"], 1),
                       "serve_3b_mixed_b32_wall_s": r["wall_s"], "serve_3b_mixed_b32_prefill_tok_s": r["prefill_tok_s"],
                       "serve_3b_mixed_b32_decode_tok_s": r["decode_tok_s"],
                       "serve_3b_mixed_b32_decode_frac": r.get("decode_hbm_frac"),
                       "serve_3b_mixed_b32_pages_reused": r["pages_reused"],
                       "serve_3b_mixed_b32_preemptions": r["preemptions"]})
        gc.collect()
        torch.cuda.empty_cache()
        long = sweep.build_parser().parse_args(
            ["--prompt-len", "8192", "--new-tokens", "512", "--max-batch-tokens", "8192", "--chunk-size", "2048",
             "--reserve-policy", "pow2", "--tune-gemm"])
        for mode in ("paged", "contiguous"):
            r = sweep.run_one(long, "8b", 64, mode)
            key = f"serve_8b_b64_ctx8704_{mode}"
            points.update({key + "_decode_tok_s": r["decode_tok_s"], key + "_decode_frac": r.get("decode_hbm_frac"),
                           key + "_prefill_tok_s": r["prefill_tok_s"], key + "_wall_s": r["wall_s"],
                           key + "_kv_tokens_reserved": r["peak_kv_tokens_reserved"],
                           key + "_kv_tokens_live": r["peak_kv_tokens_live"],
                           key + "_reserved_over_live": r["reserved_over_live"],
                           key + "_pages_reused": r["pages_reused"], key + "_preemptions": r["preemptions"],
                           key + "_fragmentation_failures": r["fragmentation_failures"]})
            gc.collect()
            torch.cuda.empty_cache()

    out = {
        "metric": f"decode tok/s at batch {args.batch} (context {ctx}), Llama-3.2-1B shape", "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic: random weights N(0,0.02), seeded uniform token ids (prompts are prefilled, then decoded)",
        "config": {"model": "llama-3.2-1b-shape", "global_batch": args.batch, "seq_len": ctx,
                   "parallelism": "single-gpu", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "page_size": PAGE, "prefill_tokens": PREFILL_TOKENS, "tied_embeddings": True,
                   "rope": "llama3 factor 32", "sampling": "greedy on device"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_gb": round(step_bytes / 1e9, 3),
                     "probed_read_stream": round(probed_gbs, 1), "frac_of_probed": round(achieved / probed_gbs, 4)},
        "points": points,
    }
    if kernel_ms is not None:
        out["kernel_ms"] = kernel_ms
        for run, classes in kernel_ms.items():          # and flat, beside the other points
            for cls, ms in classes.items():
                name = "".join(c if c.isalnum() else "_" for c in cls).strip("_")
                while "__" in name:
                    name = name.replace("__", "_")
                points[f"kclass_{run}_{name}_ms"] = ms
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
