"""The whole engine at real layer widths against the plain implementation.

Two layers of each of the three shapes the presets name (the widths, head counts, head sizes, vocabulary and
frequency scaling of the 3B, 1B and 8B models; fewer layers, so that the plain implementation on the CPU takes
seconds), with seeded random weights, in float32 and in bfloat16.  At these widths the engine takes the paths the
tiny models never reach together: the few-row products with fused epilogues at K of 3,072 to 14,336 in their
16-wave shapes, the BLAS library from 17 rows on, the matrix-core attention of head sizes 128 and 64 with groups
of 3 and 4, key splits of 1 to 8 workgroups, a vocabulary of 128,256 (reference:
``benchmarks/bench_paged_cudagraph.py:236-264`` compares its fast path's logits at the real model the same way).
"""

import copy

import pytest
import torch

import plain_llama as plain
from helpers import TOLERANCE, random_tokens, rel_err
from simple_inference_amd import preset
from simple_inference_amd.engine import StepEntry

pytestmark = pytest.mark.gpu

SHAPES = {"3b": "llama-3.2-3b", "1b": "llama-3.2-1b", "8b": "llama-3.1-8b"}
LAYERS = 2
PAGE = 16


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, plain config, plain weights); written and read once for all tests of the module."""
    made = {}

    def get(name):
        if name not in made:
            from simple_inference_amd.config import EngineConfig
            from simple_inference_amd.engine import build_model
            from simple_inference_amd.weights import random_tensors, write_model_folder
            cfg = preset(SHAPES[name])
            cfg["num_hidden_layers"] = LAYERS
            cfg["max_position_embeddings"] = 8192
            model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
            tensors = random_tensors(model.expected_tensors(), seed=7, std=0.02, gain_std=0.1, device="cuda:0")
            folder = write_model_folder(tmp_path_factory.mktemp(f"real_{name}"), mcfg.to_dict(), tensors)
            del tensors
            made[name] = (folder,) + plain.read_model(folder)
        return made[name]
    return get


_plain_rows = {}


def plain_rows(models, name, tokens, rows):
    """The plain implementation's logits of ``tokens`` at ``rows`` (kept: both dtypes ask for the same)."""
    key = (name, tuple(tokens), tuple(rows))
    if key not in _plain_rows:
        _, cfg, w = models(name)
        _plain_rows[key] = plain.forward(cfg, w, tokens, rows=list(rows))
    return _plain_rows[key]


def runner_for(models, name, dtype, num_pages, max_seq_len=512, max_running=4):
    from simple_inference_amd.cache import CacheManager
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import StepRunner, model_from_folder
    from simple_inference_amd.kernels import HipKernels
    kernels = HipKernels()
    ecfg = EngineConfig(device="cuda:0", dtype=dtype, max_seq_len=max_seq_len, block_size=PAGE,
                        num_kv_blocks=num_pages, max_running=max_running)
    model, mcfg = model_from_folder(models(name)[0], ecfg, kernels)
    cache = CacheManager(model.cache_layout(), page_size=PAGE, num_pages=num_pages, max_running=max_running,
                         dtype=ecfg.torch_dtype, device="cuda:0")
    return StepRunner(model, cache, kernels, "cuda:0", max_seq_len), cache, kernels


def run_schedule(runner, cache, schedule):
    """schedule: steps of (entries, ends), an entry (request, tokens, wanted places).  {request: {position: row}}."""
    got, fed = {}, {}
    for entries, ends in schedule:
        batch = []
        for req, tokens, want in entries:
            if req not in cache.lengths:
                cache.admit(req)
                fed[req] = 0
            batch.append(StepEntry(req, tokens, want))
        logits = runner.run(batch)
        r = 0
        for req, tokens, want in entries:
            for w in want:
                got.setdefault(req, {})[fed[req] + w] = logits[r].float().cpu()
                r += 1
            fed[req] += len(tokens)
        for req in ends:
            cache.release(req)
        cache.check()
    return got


def worst_error(models, name, got, prompts, allowed=None):
    """(worst relative difference, share of places with the plain implementation's best token).  With ``allowed``
    (a relative difference) a place whose best token differs must be a tie within it: the plain implementation's
    own logits of the two tokens lie no further apart than twice the difference a logit is allowed
    (the reference demands the same best token of its two bfloat16 paths at the real model,
    ``benchmarks/bench_paged_cudagraph.py:249-264``; a random model of 128,256 tokens has near-ties that rounding
    decides, and those are the only places excused)."""
    worst, top1 = 0.0, []
    for req, rows in got.items():
        pos = sorted(rows)
        ref = plain_rows(models, name, prompts[req], pos)
        mine = torch.stack([rows[p] for p in pos])
        worst = max(worst, rel_err(mine, ref))
        same = mine.argmax(-1) == ref.argmax(-1)
        top1 += same.tolist()
        if allowed is not None:
            for r in (~same).nonzero().flatten().tolist():
                gap = float(ref[r].max() - ref[r, int(mine[r].argmax())])
                assert gap <= 2 * allowed * float(ref.abs().max()), (
                    f"{name} request {req} place {pos[r]}: best token differs and is no tie (gap {gap:.4f})")
    return worst, sum(top1) / len(top1)


def cut(tokens, sizes):
    out, i, k = [], 0, 0
    while i < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - i)
        out.append(tokens[i:i + n])
        i += n
        k += 1
    return out


def the_four_cuts(vocab):
    """One schedule with all four ways of cutting: a prompt whole; most of one in a step and its last 32 tokens one
    by one; one in portions of changing size, down to two tokens; five more mixed, up to four live, portions of
    some beside single tokens of others, in a pool so small that pages are used again."""
    prompts = {"whole": random_tokens(vocab, 200, seed=1), "tail": random_tokens(vocab, 160, seed=2),
               "cuts": random_tokens(vocab, 150, seed=3)}
    schedule = [([("whole", prompts["whole"], [0, 1, 15, 16, 17, 63, 64, 127, 128, 199])], ["whole"])]
    t = prompts["tail"]
    schedule.append(([("tail", t[:128], [127])], []))
    schedule += [([("tail", [t[i]], [0])], ["tail"] if i == 159 else []) for i in range(128, 160)]
    parts = cut(prompts["cuts"], [2, 7, 3, 16, 2, 33, 5, 64, 9])
    schedule += [([("cuts", p, list(range(len(p))))], ["cuts"] if i == len(parts) - 1 else [])
                 for i, p in enumerate(parts)]
    lengths = (70, 45, 90, 33, 64)
    mixed = {f"m{i}": random_tokens(vocab, n, seed=10 + i) for i, n in enumerate(lengths)}
    prompts.update(mixed)
    plans = {r: cut(toks[:-5], [13 + i, 2, 7, 31]) + [[x] for x in toks[-5:]] for i, (r, toks) in enumerate(mixed.items())}
    waiting, live, step = list(mixed), [], 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for r in list(live):
            if (step + int(r[1:])) % 4 == 3 and len(live) > 1:
                continue      # left out of this step
            part = plans[r].pop(0)
            entries.append((r, part, list(range(len(part)))))
            if not plans[r]:
                ends.append(r)
                live.remove(r)
        schedule.append((entries, ends))
        step += 1
    pool = sum(sorted(-(-n // PAGE) for n in lengths)[-4:]) + 1     # the four largest of the mixed ones
    return prompts, schedule, max(pool, -(-200 // PAGE))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["3b", "1b", "8b"])
def test_the_four_cuts_at_real_widths(models, name, dtype):
    vocab = models(name)[1]["vocab_size"]
    prompts, schedule, pool = the_four_cuts(vocab)
    runner, cache, _ = runner_for(models, name, dtype, num_pages=pool)
    got = run_schedule(runner, cache, schedule)
    assert sum(len(v) for v in got.values()) == 10 + 33 + 150 + 302
    worst, top1 = worst_error(models, name, got, prompts)
    backend = "hip-f32" if dtype == "float32" else "hip-bf16"
    assert worst <= TOLERANCE[backend], f"{name} {dtype}: worst relative difference {worst:.3e}"
    assert cache.free_pages() == pool
    if dtype == "float32":
        assert top1 == 1.0
    else:
        _, top1 = worst_error(models, name, got, prompts, allowed=TOLERANCE[backend])
        print(f"\n{name} bfloat16, 2 layers: worst {worst:.3e}, same best token at {top1:.1%} of 495 places")


@pytest.mark.parametrize("mode", ["float32", "bfloat16", "bfloat16-unfused"])
def test_steps_of_1_8_16_17_and_64_single_tokens_at_3b_widths(models, mode):
    """64 requests with prompts of 3 to 34 tokens decode together, then 17, 16, 8 and one of them: a step of up to
    16 rows takes this package's products (with the fused epilogues, or, in the third mode, without: product,
    rotation and cache write, norm and activation as kernels of their own), from 17 rows on the BLAS library."""
    dtype = "float32" if mode == "float32" else "bfloat16"
    _, cfg, _ = models("3b")
    vocab = cfg["vocab_size"]
    prompts = {i: random_tokens(vocab, 3 + (i * 7) % 32 + 5, seed=300 + i) for i in range(64)}
    pool = sum(-(-len(p) // PAGE) for p in prompts.values())
    runner, cache, kernels = runner_for(models, "3b", dtype, num_pages=pool, max_running=64)
    if mode.endswith("unfused"):
        kernels.fuse_norms = kernels.fuse_rope = False
    ids = list(prompts)
    schedule = []
    for first in range(0, 64, 16):      # the prompts, sixteen at a time, all but their last five tokens
        schedule.append(([(i, prompts[i][:-5], []) for i in ids[first:first + 16]], []))
    for step, group in enumerate((ids, ids[:17], ids[:16], ids[:8], ids[:1])):
        schedule.append(([(i, [prompts[i][len(prompts[i]) - 5 + step]], [0]) for i in group], []))
    got = run_schedule(runner, cache, schedule)
    assert sum(len(v) for v in got.values()) == 64 + 17 + 16 + 8 + 1
    tolerance = TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"]
    worst, top1 = worst_error(models, "3b", got, prompts, allowed=tolerance)
    assert worst <= tolerance, f"{mode}: {worst:.3e}"
    assert dtype != "float32" or top1 == 1.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_context_past_4096_tokens_crosses_every_number_of_key_splits(models, dtype):
    """One request grows to 4,100 tokens: portions bring it to just below 512, 1,024, 2,048 and 4,096 keys, and
    three single tokens then cross each of these lengths, at which the decode kernel shares a sequence between 1,
    2, 4 and 8 workgroups."""
    _, cfg, _ = models("3b")
    tokens = random_tokens(cfg["vocab_size"], 4100, seed=400)
    runner, cache, _ = runner_for(models, "3b", dtype, num_pages=-(-4100 // PAGE) + 1, max_seq_len=4352, max_running=2)
    schedule, at = [], 0
    for edge in (512, 1024, 2048, 4096):
        for part in cut(tokens[at:edge - 2], [2048]):
            schedule.append(([(0, part, [len(part) - 1])], []))
        schedule += [([(0, [tokens[i]], [0])], []) for i in range(edge - 2, edge + 2)]
        at = edge + 2
    schedule.append(([(0, tokens[at:], [len(tokens) - at - 1])], [0]))
    got = run_schedule(runner, cache, schedule)
    assert sorted(got[0])[-1] == 4099 and len(got[0]) == 4 * 4 + 4 + 1
    tolerance = TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"]
    worst, top1 = worst_error(models, "3b", got, {0: tokens}, allowed=tolerance)
    assert worst <= tolerance, f"{dtype}: {worst:.3e}"
    assert dtype != "float32" or top1 == 1.0


# ---- the headline model at its full depth ------------------------------------------------------------------------

FULL_DEPTH = {}


@pytest.fixture(scope="module")
def full_depth(tmp_path_factory):
    """The 3B shape with all its layers: the model folder, and the plain implementation's weights in float64 on the
    GPU (the plain implementation is elementary torch and runs wherever its tensors lie; in float64 no question
    of a reduced-precision matrix mode arises)."""
    if not FULL_DEPTH:
        from simple_inference_amd.config import EngineConfig
        from simple_inference_amd.engine import build_model
        from simple_inference_amd.weights import random_tensors, write_model_folder
        cfg = preset(SHAPES["3b"])
        cfg["max_position_embeddings"] = 8192
        model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
        tensors = random_tensors(model.expected_tensors(), seed=11, std=0.02, gain_std=0.1, device="cuda:0")
        folder = write_model_folder(tmp_path_factory.mktemp("full_3b"), mcfg.to_dict(), tensors)
        del tensors
        from safetensors import safe_open
        weights = {}
        with safe_open(str(folder / "model.safetensors"), framework="pt") as f:     # tensor by tensor: the host
            for key in f.keys():                                                    # never holds the model in float64
                weights[key] = f.get_tensor(key).to("cuda:0").double()
        FULL_DEPTH.update(folder=folder, cfg=plain.read_config(folder), weights=weights, exact={}, rounded={})
    yield FULL_DEPTH
    FULL_DEPTH.clear()      # 26 GB of float64 weights go back when the module's tests are done


def _plain_at_full_depth(fd, tokens, rows, rounded):
    key = (tuple(tokens), tuple(rows))
    kept = fd["rounded" if rounded else "exact"]
    if key not in kept:
        fn = plain.forward_as_the_reference_rounds if rounded else plain.forward
        kept[key] = fn(fd["cfg"], fd["weights"], tokens, rows=list(rows)).float().cpu()
    return kept[key]


def _rms(a, b):
    a, b = a.double(), b.double()
    return float(((a - b).pow(2).mean() / b.pow(2).mean()).sqrt())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_four_cuts_at_full_depth(full_depth, dtype):
    """All 28 layers of the headline shape, seeded random weights with gains of 1 + N(0, 0.1), against the plain
    implementation in float64 under the four ways of cutting the work (reference: its fast path against its plain
    one at the real model, ``benchmarks/bench_paged_cudagraph.py:236-264``).

    float32: the tolerance of the tiny models holds at depth too (only the order of additions differs).
    bfloat16: rounding errors grow with depth by the model's own sensitivity, which no constant chosen at two
    layers knows.  The bound is therefore measured on the model itself: the plain implementation is run a second
    time with every intermediate result rounded to bfloat16 where the reference's bfloat16 model rounds
    (``plain.forward_as_the_reference_rounds``), and the engine may lie no further from exact arithmetic than that
    correct bfloat16 computation does, over the same places: in the largest difference of a logit and in the
    root mean square of all differences, both relative to the size of the logits.  A place where the engine's
    best token is not the plain implementation's must be a tie within twice that bound."""
    fd = full_depth
    vocab = fd["cfg"]["vocab_size"]
    prompts, schedule, pool = the_four_cuts(vocab)
    from simple_inference_amd.cache import CacheManager
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import StepRunner, model_from_folder
    from simple_inference_amd.kernels import HipKernels
    kernels = HipKernels()
    ecfg = EngineConfig(device="cuda:0", dtype=dtype, max_seq_len=512, block_size=PAGE, num_kv_blocks=pool, max_running=4)
    model, mcfg = model_from_folder(fd["folder"], ecfg, kernels)
    assert mcfg.num_hidden_layers == 28 == len(model.order)
    cache = CacheManager(model.cache_layout(), page_size=PAGE, num_pages=pool, max_running=4,
                         dtype=ecfg.torch_dtype, device="cuda:0")
    got = run_schedule(StepRunner(model, cache, kernels, "cuda:0", 512), cache, schedule)
    assert sum(len(v) for v in got.values()) == 10 + 33 + 150 + 302 and cache.free_pages() == pool
    del model
    mine, exact, rounded = [], [], []
    for req, rows in got.items():
        pos = sorted(rows)
        mine.append(torch.stack([rows[p] for p in pos]))
        exact.append(_plain_at_full_depth(fd, prompts[req], pos, rounded=False))
        if dtype == "bfloat16":
            rounded.append(_plain_at_full_depth(fd, prompts[req], pos, rounded=True))
    mine, exact = torch.cat(mine), torch.cat(exact)
    worst, rms = rel_err(mine, exact), _rms(mine, exact)
    same = mine.argmax(-1) == exact.argmax(-1)
    if dtype == "float32":
        print(f"\n3b float32, 28 layers: worst {worst:.3e}, rms {rms:.3e}, same best token at {float(same.float().mean()):.1%}")
        assert worst <= TOLERANCE["hip-f32"], worst
        assert bool(same.all())
        return
    rounded = torch.cat(rounded)
    allowed_worst, allowed_rms = rel_err(rounded, exact), _rms(rounded, exact)
    same_rounded = rounded.argmax(-1) == exact.argmax(-1)
    print(f"\n3b bfloat16, 28 layers: worst {worst:.3e} (bound {allowed_worst:.3e}), rms {rms:.3e} (bound {allowed_rms:.3e}), "
          f"same best token at {float(same.float().mean()):.1%} of {len(same)} places "
          f"(the rounded plain implementation: {float(same_rounded.float().mean()):.1%})")
    assert worst <= allowed_worst and rms <= allowed_rms
    scale = float(exact.abs().max())
    for r in (~same).nonzero().flatten().tolist():
        gap = float(exact[r].max() - exact[r, int(mine[r].argmax())])
        assert gap <= 2 * allowed_worst * scale, f"place {r}: best token differs and is no tie (gap {gap:.4f})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_of_a_long_prompt_are_read_again_by_a_short_one_at_8b_widths(models, dtype):
    """Prefix reuse at real widths: a prompt of 2,048 tokens fills its pages in one step of 2,048 rows (the library's
    products, the prefill attention shape for long prompts, rotation and cache write of long steps); a second
    request with the same first 1,024 tokens and 17 of its own then runs those 17 rows only, reading 64 pages the
    first one wrote, and goes on decoding.  Its tokens are the plain implementation's (which knows no cache),
    apart from ties within rounding in bfloat16."""
    from simple_inference_amd import Engine, EngineConfig
    folder, cfg, w = models("8b")
    vocab = cfg["vocab_size"]
    first = random_tokens(vocab, 2048, seed=500)
    second = first[:1024] + random_tokens(vocab, 17, seed=501)
    engine = Engine.from_folder(folder, EngineConfig(
        device="cuda:0", dtype=dtype, max_seq_len=2304, block_size=PAGE, max_running=2, chunk_tokens=2048, eos_id=-1,
        use_prefix_cache=True))
    a = engine.add_request(first, max_new_tokens=2)
    engine.run()
    b = engine.add_request(second, max_new_tokens=6)
    engine.run()
    assert a.cached_prefix_len == 0 and b.cached_prefix_len == 1024
    assert engine.stats["prefill_tokens"] == 2048 + 17
    tolerance = TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"]
    w = {k: v.to("cuda:0") for k, v in w.items()}      # the plain implementation runs where its tensors lie
    for req in (a, b):
        tokens = list(req.prompt_tokens)
        for got in req.generated:
            logits = plain.forward(cfg, w, tokens, rows=[len(tokens) - 1])[0].cpu()
            want = int(logits.argmax())
            gap = float(logits[want] - logits[got])
            assert got == want or (dtype == "bfloat16" and gap <= 2 * tolerance * float(logits.abs().max())), (got, want, gap)
            tokens.append(got)
    engine.cache.check()
