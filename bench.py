"""Measurement: decode tokens a second and prefill tokens a second at the Llama-3.2-3B shape.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A "step" is one decode step of the engine (scheduler, one call of the
step function over the batch, sampling).  The default run has the layer sizes of the 3B shape
(28 layers, hidden 3072, 24 query / 8 key-value heads of 128, feed-forward 8192, vocabulary
128256, tied head) with seeded random bfloat16 weights, a batch of 8 requests, each with a
2,048-token context of uniform-random token ids, and a context limit of 4,096.  Beside the
headline it reports the prefill of one 2,048-token prompt (one step of the engine), decode at
batch 1 and 64, how close the decode step comes to the HBM roofline (the published 8 TB/s and
what a plain streaming read measures on the card) and the prefill to the matrix-core peak, and
a check of the logits: one decode step of the bfloat16 engine against the float32 engine built
from the same seed, on the same tokens.  With the default 256 steps every request decodes from
2,048 to 2,304 tokens of context.

Two further workloads run whole request streams through the scheduler (``--workload``):
``continuous``: 128 requests at the 1B shape, prompts of 64..2,048 and outputs of 32..512 tokens,
prompts cut into portions of 512; ``shared-prefix``: 64 requests at the 8B shape with one
1,024-token prefix, 256 tokens of their own and 256 decoded tokens each, with and without
prefix reuse.  They print one JSON line of their own kind.

The engine runs on one GPU; asked for more it says so and exits with 2.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

import torch

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense matrix-core peaks, published

# How far the bfloat16 engine's logits may lie from the float32 engine's, as the largest difference of a logit
# relative to the largest logit.  A correct bfloat16 computation of a model errs by an amount that grows with its
# depth and follows the model's own sensitivity, so the bound is measured, not guessed: the plain implementation
# under tests/, run in float64 with every intermediate result rounded where the reference's bfloat16 model rounds,
# differs from exact arithmetic by 5.0e-2 at all 28 layers of the 3B shape with weights of this distribution
# (tests/test_real_sizes_gpu.py measures it and holds the engine to it on 495 places).  For a run with another
# number of layers the bound is scaled by the root of the depth, as independent rounding errors add up.  A run
# whose logits differ by more, or that picks another best token where the float32 logits do not tie within twice
# the bound, ends with status 3.
def logit_bound(layers: int) -> float:
    return 5.0e-2 * (layers / 28) ** 0.5


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="tokens each request holds before decoding")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--preset", default="llama-3.2-3b")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--block-size", type=int, default=None)
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--points", default="1,64,16,17", help="further decode batch sizes to report, comma separated")
    ap.add_argument("--no-further-points", action="store_true",
                    help="only the headline and --points: no long contexts, other prompt lengths or request streams")
    ap.add_argument("--chunk-tokens", type=int, default=512, help="most tokens a step of the stream workloads runs")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-check", action="store_true", help="skip the comparison of logits with the float32 engine")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--temperature", type=float, default=0.0, help="sampling of the decode measurement (0: greedy)")
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "shared-prefix"])
    ap.add_argument("--max-running", type=int, default=64, help="request slots of the stream workloads")
    return ap.parse_args(argv)


def build_engine(args, max_batch, total_len):
    from simple_inference_amd import Engine, EngineConfig, preset

    cfg = preset(args.preset)
    layers_full = cfg["num_hidden_layers"]
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    kw = {}
    if args.block_size:
        kw["block_size"] = args.block_size
    ecfg = EngineConfig(
        max_running=max_batch, max_seq_len=max(4096, -(-total_len // 1024) * 1024), dtype=args.dtype, chunk_tokens=max(2048, args.prefill_tokens),
        eos_id=-1, use_graphs=not args.no_graphs, device="cuda:0", **kw)
    ecfg.num_kv_blocks = max_batch * (-(-total_len // ecfg.block_size)) + 8
    engine = Engine.from_random(cfg, seed=args.seed, engine_cfg=ecfg, std=0.02, generate_on_device=True)
    return engine, cfg, layers_full


def matmul_params(mc):
    """Weights of the matrix products of one forward pass of one token (head included once)."""
    q = mc.num_attention_heads * mc.head_dim
    kv = mc.num_key_value_heads * mc.head_dim
    per_layer = mc.hidden_size * (q + 2 * kv) + q * mc.hidden_size + 3 * mc.hidden_size * mc.intermediate_size
    return mc.num_hidden_layers * per_layer, mc.vocab_size * mc.hidden_size


def random_prompt(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def decode_allowance(engine_or_chunk, batch, context):
    """Tokens a request may decode while the other prompts of its batch are still being run, and two to spare."""
    chunk = engine_or_chunk if isinstance(engine_or_chunk, int) else engine_or_chunk.cfg.chunk_tokens
    return batch * (-(-context // chunk)) + 2


def measure_decode(engine, batch, context, steps, warmup, seed=0, sampling=(0.0, 0, 1.0)):
    """(seconds per step, mean context over the timed steps) with ``batch`` requests decoding."""
    from simple_inference_amd import SamplingParams

    engine.reset()
    vocab = engine.model.vocab_size
    temperature, top_k, top_p = sampling
    reqs = [engine.add_request(random_prompt(vocab, context, seed + i), params=SamplingParams(
        temperature=temperature, top_k=top_k, top_p=top_p, seed=seed + i,
        max_new_tokens=warmup + steps + decode_allowance(engine, batch, context), ignore_eos=True)) for i in range(batch)]
    while any(r.num_generated == 0 for r in reqs):   # prefill every prompt
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    ctx0 = sum(r.context_len for r in reqs) / batch
    before = [r.num_generated for r in reqs]
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    ctx1 = sum(r.context_len for r in reqs) / batch
    assert all(r.num_generated == b + steps for r, b in zip(reqs, before)), "a request did not decode in every step"
    engine.reset()
    return dt, (ctx0 + ctx1) / 2


def measure_prefill(engine, tokens, repeats=3, seed=100):
    """(mean, best) seconds of the one step that runs a prompt of ``tokens`` tokens, over ``repeats`` runs."""
    from simple_inference_amd import SamplingParams

    vocab = engine.model.vocab_size
    times = []
    for i in range(repeats + 1):   # the first is warmup
        engine.reset()
        engine.add_request(random_prompt(vocab, tokens, seed + i), params=SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        if i > 0:
            times.append(time.perf_counter() - t0)
    engine.reset()
    return sum(times) / len(times), min(times)


def logits_check(engine, cfg, seed, batch=4, context=512):
    """One decode step of the serving engine against a float32 engine with the same weights (same seed), on the same
    tokens: the largest difference of the logits relative to their size, and how often the best token is the same
    (the reference checks its fast path that way at the real model: ``benchmarks/bench_paged_cudagraph.py:236-264``).
    ``ok`` says whether the difference is within ``logit_bound`` and every differing best token a tie within
    twice that bound."""
    from simple_inference_amd import Engine, EngineConfig
    from simple_inference_amd.engine import StepEntry

    vocab = engine.model.vocab_size
    prompts = [random_prompt(vocab, context, seed + 500 + i) for i in range(batch)]
    exact = Engine.from_random(cfg, seed=seed, engine_cfg=EngineConfig(
        max_running=batch, max_seq_len=context + 16, dtype="float32", chunk_tokens=batch * context, eos_id=-1,
        use_graphs=False, device="cuda:0", block_size=engine.cfg.block_size), std=0.02, generate_on_device=True)

    def last_logits(eng):
        eng.reset()
        ids = [10 ** 6 + i for i in range(batch)]
        for i in ids:
            eng.cache.admit(i)
        eng.runner.run([StepEntry(i, p[:-1], []) for i, p in zip(ids, prompts)])
        logits = eng.runner.run([StepEntry(i, [p[-1]], [0]) for i, p in zip(ids, prompts)]).float()
        eng.reset()
        return logits
    got, want = last_logits(engine), last_logits(exact)
    del exact
    torch.cuda.empty_cache()
    scale = float(want.abs().max())
    rel = float((got - want).abs().max()) / scale
    rms = float(((got - want).double().pow(2).mean() / want.double().pow(2).mean()).sqrt())
    best, best_exact = got.argmax(-1), want.argmax(-1)
    bound = logit_bound(engine.model_cfg.num_hidden_layers)
    gaps = [float(want[r, best_exact[r]] - want[r, best[r]]) for r in range(batch)]
    ties = all(g <= 2 * bound * scale for g in gaps)
    return {"against": "float32 engine, same seed and tokens", "batch": batch, "context": context,
            "rel_err": round(rel, 5), "rms_err": round(rms, 5), "bound": round(bound, 5),
            "top1_agree": float((best == best_exact).float().mean()), "top1_agree_or_tie": 1.0 if ties else 0.0,
            "ok": bool(rel <= bound and ties)}


def run_stream(preset_name, requests, max_running, max_seq_len, prefix_cache, args, chunk_tokens=None):
    """Queues all requests at once and steps the engine dry; returns the figures of the run."""
    from simple_inference_amd import Engine, EngineConfig, SamplingParams, preset

    ecfg = EngineConfig(max_running=max_running, max_seq_len=max_seq_len,
                        chunk_tokens=chunk_tokens or args.chunk_tokens, dtype=args.dtype,
                        eos_id=-1, use_graphs=not args.no_graphs, use_prefix_cache=prefix_cache, device="cuda:0")
    engine = Engine.from_random(preset(preset_name), seed=args.seed, engine_cfg=ecfg, std=0.02,
                                generate_on_device=True)
    def one_pass():
        engine.reset()
        for key in engine.stats:
            engine.stats[key] = 0
        handles = [engine.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True))
                   for p, n in requests]
        first, last = {}, {}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while engine.has_work():
            emitted = engine.step()          # the tokens have reached the host when it returns
            now = time.perf_counter() - t0
            for rid in emitted:
                first.setdefault(rid, now)
                last[rid] = now
        torch.cuda.synchronize()
        sec = time.perf_counter() - t0
        assert all(len(h.generated) == n for h, (_, n) in zip(handles, requests))
        engine.cache.check()
        return handles, first, last, sec

    one_pass()   # untimed: the graphs this stream replays are captured here, as a server's warm-up captures them
    handles, first, last, sec = one_pass()
    by_id = {h.id: h for h in handles}

    def percentiles(values):
        v = sorted(values)
        return {f"p{q}": round(v[min(len(v) - 1, int(len(v) * q / 100))] * 1e3, 2) for q in (50, 90, 99)}
    ttft = [first[i] for i in by_id]                       # every request is queued at time 0
    tpot = [(last[i] - first[i]) / (len(by_id[i].generated) - 1) for i in by_id if len(by_id[i].generated) > 1]
    check = stream_check(engine, [(list(h.prompt_tokens), list(h.generated)) for h in handles])
    out = {"seconds": round(sec, 3), "steps": engine.stats["steps"], "prompt_tokens": sum(len(p) for p, _ in requests),
           "prefill_tokens_run": engine.stats["prefill_tokens"], "generated_tokens": engine.stats["decode_tokens"] + len(requests),
           "generated_tok_s": round(sum(n for _, n in requests) / sec, 1),
           "ttft_ms": percentiles(ttft), "tpot_ms": percentiles(tpot), "check": check}
    del engine
    torch.cuda.empty_cache()
    return out


def stream_check(engine, finished, sample=4, last=8):
    """Were the stream's tokens the right ones?  A few of its requests are run again alone, whole (prompt and what
    the stream generated for it, in one step), and the stream's last tokens are compared with what that run would
    choose at the same places: equal, or tied with it within bfloat16 rounding (the stream met those tokens in
    steps of other sizes, which the BLAS library multiplies in another order).  Two logits count as tied if they
    are no further apart than twice what the reference allows one logit of its fast path to be from its plain
    one at full size (``benchmarks/bench_paged_cudagraph.py:236-264``: 0.15 + 0.05 |logit|); a token from a wrong
    page or a wrong row would be several units away."""
    from simple_inference_amd.engine import StepEntry

    engine.reset()
    picks = sorted({(len(finished) - 1) * i // max(sample - 1, 1) for i in range(sample)})
    same = close = total = 0
    for n, i in enumerate(picks):
        prompt, generated = finished[i]
        k = min(last, len(generated))
        tokens = prompt + generated[:-1]
        places = [len(tokens) - k + j for j in range(k)]          # the places that chose the last k tokens
        rid = 10 ** 6 + n
        engine.cache.admit(rid)
        logits = engine.runner.run([StepEntry(rid, tokens, places)]).float()
        engine.cache.release(rid)
        for row, token in zip(logits, generated[-k:]):
            best = int(row.argmax())
            total += 1
            same += best == token
            close += best == token or float(row[best] - row[token]) <= 2 * (0.15 + 0.05 * abs(float(row[best])))
    assert close == total, f"{total - close} of {total} checked tokens are not what a solo run would choose"
    return {"requests": len(picks), "tokens": total, "same_as_solo": same, "tied_within_rounding": close - same}


def continuous_requests(seed):
    """128 requests of the 1B workload: prompts of 64..2,048 and outputs of 32..512 tokens, uniform."""
    import random

    from simple_inference_amd import preset
    rng = random.Random(seed)
    vocab = preset("llama-3.2-1b")["vocab_size"]
    return [([rng.randrange(vocab) for _ in range(rng.randint(64, 2048))], rng.randint(32, 512)) for _ in range(128)]


def shared_prefix_requests(seed):
    """64 requests of the 8B workload: one 1,024-token prefix, 256 tokens of their own, 256 decoded tokens each."""
    import random

    from simple_inference_amd import preset
    rng = random.Random(seed)
    vocab = preset("llama-3.1-8b")["vocab_size"]
    shared = [rng.randrange(vocab) for _ in range(1024)]
    return [(shared + [rng.randrange(vocab) for _ in range(256)], 256) for _ in range(64)]


def stream_workload(args):
    if args.workload == "continuous":
        name = "llama-3.2-1b"
        run = run_stream(name, continuous_requests(args.seed), args.max_running, 4096, False, args)
        line = {"metric": "generated tok/s, continuous batching of 128 requests (1B shape)", "value": run["generated_tok_s"],
                "run": run}
    else:
        name = "llama-3.1-8b"
        requests = shared_prefix_requests(args.seed)
        reuse = run_stream(name, requests, args.max_running, 8192, True, args)
        plain = run_stream(name, requests, args.max_running, 8192, False, args)
        line = {"metric": "generated tok/s, 64 requests with a shared 1,024-token prefix (8B shape), prefix reuse on",
                "value": reuse["generated_tok_s"], "run": reuse, "without_reuse": plain}
    line.update({"unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "warmup": "one untimed pass of the same stream", "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
                 "data": "synthetic (seeded random weights N(0, 0.02) and uniform-random token ids)",
                 "config": {"model": name + "-shape", "max_running": args.max_running, "chunk_tokens": args.chunk_tokens,
                            "graphs": not args.no_graphs}})
    print(json.dumps(line), flush=True)
    return 0


def further_points(args, pts, config, layer_w, head_w, el):
    """What the headline leaves out, at sizes a server meets: the same model with contexts of 8,192 and 32,768 tokens
    and a prompt of 8,192 (an engine of its own with a context limit of 33,792), and the two request streams of the
    other shapes, each through scheduler, step function and sampler, with a sample of its tokens checked against
    solo runs."""
    import copy
    from simple_inference_amd import Engine, EngineConfig, preset

    long_args = copy.copy(args)
    long_limit = 32768 + 1024
    cfg = preset(args.preset)
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    steps, warmup = min(args.steps, 32), min(args.warmup, 4)
    ecfg = EngineConfig(max_running=8, max_seq_len=long_limit, dtype=args.dtype, chunk_tokens=8192, eos_id=-1,
                        use_graphs=not args.no_graphs, device="cuda:0")
    ecfg.num_kv_blocks = 8 * (-(-long_limit // ecfg.block_size)) + 8
    engine = Engine.from_random(cfg, seed=args.seed, engine_cfg=ecfg, std=0.02, generate_on_device=True)
    mc = engine.model_cfg
    config["long_context_limit"] = long_limit
    for context in (8192, 32768):
        dt, ctx = measure_decode(engine, 8, context, steps, warmup, args.seed)
        gbs = ((layer_w + head_w) * el + 8 * ctx * mc.kv_bytes_per_token(el)) / dt / 1e9
        pts[f"decode_b8_ctx{context}"] = round(8 / dt, 2)
        pts[f"decode_b8_ctx{context}_hbm_frac"] = round(gbs / PEAK_HBM_GBS, 4)
    if not args.no_prefill:
        T = 8192
        sec, _ = measure_prefill(engine, T, repeats=2)
        flops = 2 * layer_w * T + 2 * head_w + mc.num_hidden_layers * 4 * mc.num_attention_heads * mc.head_dim * T * (T + 1) / 2
        pts["prefill_8192"] = round(T / sec, 1)
        pts["prefill_8192_frac"] = round(flops / sec / PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"], 4)
    del engine
    torch.cuda.empty_cache()
    if args.preset != "llama-3.2-3b" or args.layers is not None:
        return      # the streams belong to the default run
    run = run_stream("llama-3.2-1b", continuous_requests(args.seed), 64, 4096, False, args)
    config["stream_1b"] = f"llama-3.2-1b-shape, 128 requests, max_running 64, chunk_tokens {args.chunk_tokens}"
    pts["stream_1b_tok_s"] = run["generated_tok_s"]
    pts["stream_1b_seconds"] = run["seconds"]
    pts["stream_1b_tpot_p50_ms"] = run["tpot_ms"]["p50"]
    pts["stream_1b_tpot_p99_ms"] = run["tpot_ms"]["p99"]
    pts["stream_1b_checked_tokens"] = run["check"]["tokens"]
    # the same stream with portions of 2,048 tokens: fewer, fuller steps (a step of 512 rows costs 1.8 times as much a
    # token as one of 2,048), paid for by the decoding requests that wait behind them
    wide = run_stream("llama-3.2-1b", continuous_requests(args.seed), 64, 4096, False, args, chunk_tokens=2048)
    pts["stream_1b_chunk2048_tok_s"] = wide["generated_tok_s"]
    pts["stream_1b_chunk2048_tpot_p50_ms"] = wide["tpot_ms"]["p50"]
    pts["stream_1b_chunk2048_tpot_p99_ms"] = wide["tpot_ms"]["p99"]
    requests = shared_prefix_requests(args.seed)
    config["prefix_8b"] = f"llama-3.1-8b-shape, 64 requests, prefix 1024, max_running 64, chunk_tokens {args.chunk_tokens}"
    reuse = run_stream("llama-3.1-8b", requests, 64, 8192, True, args)
    plain = run_stream("llama-3.1-8b", requests, 64, 8192, False, args)
    pts["prefix_8b_seconds"] = reuse["seconds"]
    pts["prefix_8b_seconds_without"] = plain["seconds"]
    pts["prefix_8b_prompt_tokens_run"] = reuse["prefill_tokens_run"]
    pts["prefix_8b_checked_tokens"] = reuse["check"]["tokens"] + plain["check"]["tokens"]


def main(argv=None):
    args = parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    if args.workload != "decode":
        return stream_workload(args)
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    chunk = max(2048, args.prefill_tokens)
    total_len = max(args.context + args.warmup + args.steps + decode_allowance(chunk, max_batch, args.context),
                    args.prefill_tokens + 2)
    engine, cfg, layers_full = build_engine(args, max_batch, total_len)
    mc = engine.model_cfg
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    el = 2 if args.dtype == "bfloat16" else 4
    layer_w, head_w = matmul_params(mc)

    def decode_point(batch):
        dt, ctx = measure_decode(engine, batch, args.context, args.steps, args.warmup, args.seed,
                                 (args.temperature, args.top_k, args.top_p))
        bytes_read = (layer_w + head_w) * el + batch * ctx * mc.kv_bytes_per_token(el)
        return dt, batch / dt, bytes_read / dt / 1e9

    dt, tok_s, gbs = decode_point(args.batch)
    line = {
        "metric": (f"decode tok/s at batch 8; prefill tok/s at {args.prefill_tokens:,} tokens "
                   f"({args.preset.rsplit('-', 1)[-1].upper()}, {dt_name})")
                  if args.batch == 8 and not args.no_prefill else f"decode tok/s at batch {args.batch}",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt_name, "data": "synthetic (seeded random weights N(0, 0.02) and uniform-random token ids)",
        "config": {
            "model": args.preset + "-shape", "layers": mc.num_hidden_layers, "layers_full": layers_full,
            "hidden": mc.hidden_size, "heads": mc.num_attention_heads, "kv_heads": mc.num_key_value_heads,
            "head_dim": mc.head_dim, "intermediate": mc.intermediate_size, "vocab": mc.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "context_limit": engine.cfg.max_seq_len,
            "page_size": engine.cfg.block_size, "graphs": engine.graphs is not None, "parallelism": "single GPU",
            "prefill_step_tokens": args.prefill_tokens,
            "sampling": "greedy" if args.temperature == 0 else f"T={args.temperature} k={args.top_k} p={args.top_p}",
        },
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4)},
    }
    measured = engine.kernels.measured_read_bandwidth()
    line["roofline"]["measured_copy"] = round(measured, 1)        # a plain streaming read on this card
    line["roofline"]["frac_of_measured"] = round(gbs / measured, 4)
    if not args.no_prefill:
        T = args.prefill_tokens
        sec, best = measure_prefill(engine, T)
        attn_flops = mc.num_hidden_layers * 4 * mc.num_attention_heads * mc.head_dim * T * (T + 1) / 2
        flops = 2 * layer_w * T + 2 * head_w * 1 + attn_flops
        line["prefill"] = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                           "frac": round(flops / sec / PEAK_FLOPS[dt_name], 4), "best_ms": round(best * 1e3, 3)}
    pts = {}
    for b in points:
        _, p_tok_s, p_gbs = decode_point(b)
        pts[f"decode_b{b}"] = round(p_tok_s, 2)
        pts[f"decode_b{b}_hbm_frac"] = round(p_gbs / PEAK_HBM_GBS, 4)
    if not args.no_check and args.dtype == "bfloat16":
        line["check"] = logits_check(engine, cfg, args.seed)
    if not args.no_further_points and not args.no_prefill:
        sec, _ = measure_prefill(engine, 512)        # the default portion of a prompt (chunk_tokens of the engine)
        pts["prefill_512"] = round(512 / sec, 1)
        pts["prefill_512_ms"] = round(sec * 1e3, 3)
    if not args.no_further_points:
        del engine
        torch.cuda.empty_cache()
        further_points(args, pts, line["config"], layer_w, head_w, el)
    if pts:
        line["points"] = pts
    print(json.dumps(line), flush=True)
    if "check" in line and not line["check"]["ok"]:
        print(f"bench.py: the bfloat16 logits are further from the float32 engine's than a correct bfloat16 "
              f"computation may be: {line['check']}", file=sys.stderr, flush=True)
        return 3
    return 0


if __name__ == "__main__":
    sys.exit(main())
