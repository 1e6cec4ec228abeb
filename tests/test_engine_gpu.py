"""The engine on the GPU: greedy generation through the entry points, graph replay, sampling."""

import pytest
import torch

import plain_llama as plain
from helpers import TINIES, TOLERANCE, random_tokens, rel_err, write_tiny_model
from simple_inference_amd import Engine, EngineConfig, RequestState, SamplingParams
from simple_inference_amd.engine import StepEntry
from simple_inference_amd.sampling import uniform_for

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {n: write_tiny_model(tmp_path_factory.mktemp(f"eng_{n}"), t, seed=51) for n, t in TINIES.items()}


def engine(folder, tiny, dtype, **kw):
    base = dict(device="cuda:0", dtype=dtype, max_seq_len=256, block_size=tiny.page_size, max_running=4,
                chunk_tokens=24, eos_id=-1)
    base.update(kw)
    return Engine.from_folder(folder, EngineConfig(**base))


def greedy_matches_plain(folder, prompt, generated, dtype):
    """Every generated token is the plain implementation's argmax, or (bfloat16) one whose logit ties with it."""
    cfg, w = plain.read_model(folder)
    toks = list(prompt)
    for got in generated:
        logits = plain.forward(cfg, w, toks)[-1]
        want = int(logits.argmax())
        if got != want:
            margin = float(logits[want] - logits[got])
            assert dtype == "bfloat16" and margin <= 2.5e-2 * float(logits.abs().max()), (got, want, margin)
        toks.append(got)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINIES))
def test_greedy_generation_through_the_entry_points(folders, name, dtype):
    tiny = TINIES[name]
    vocab = tiny.config["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=60 + i) for i, n in enumerate((1, 17, 40, 70))]
    eng = engine(folders[name], tiny, dtype)
    reqs = [eng.add_request(p, max_new_tokens=8) for p in prompts]
    eng.run()
    for p, r in zip(prompts, reqs):
        assert r.state is RequestState.FINISHED and r.num_generated == 8
        greedy_matches_plain(folders[name], p, r.generated, dtype)
    assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()
    # the streaming entry point gives the same tokens as the batch did
    solo = engine(folders[name], tiny, dtype, max_running=1)
    assert list(solo.generate(prompts[2], max_new_tokens=8, temperature=0.0)) == reqs[2].generated


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager_on_every_replay(folders, dtype):
    """Replayed steps against the same steps run eagerly, with eager work and synchronisation between
    replays, several batch buckets and a growing context."""
    tiny = TINIES["b"]
    vocab = tiny.config["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=70 + i) for i, n in enumerate((5, 33, 12))]
    eager = engine(folders["b"], tiny, dtype, use_graphs=False)
    graphed = engine(folders["b"], tiny, dtype, use_graphs=True)
    ra = [eager.add_request(p, max_new_tokens=20 - 4 * i) for i, p in enumerate(prompts)]
    rb = [graphed.add_request(p, max_new_tokens=20 - 4 * i) for i, p in enumerate(prompts)]
    while eager.has_work() or graphed.has_work():
        a, b = eager.step(), graphed.step()
        torch.cuda.synchronize()
        assert list(a.values()) == list(b.values())
    assert [r.generated for r in ra] == [r.generated for r in rb]
    assert graphed.graphs.replays >= 15 and len(graphed.graphs._made) >= 2       # buckets 4, 2, 1 as requests end


def test_graph_replay_of_many_rows_equals_eager_on_every_replay(folders):
    """Twenty and more requests: the products of a replayed step then go to the BLAS library, whose launches are
    captured with this package's.  Every replay's logits against the same step run eagerly on a twin engine, with
    eager work and synchronisation between the replays (a captured memset would show from the second replay on).
    The eager twin runs where a graph's shapes are settled (``recurring_shapes``), so that it multiplies with the
    library algorithms the graph recorded: the same kernels and library calls, replayed or not, give the same
    bits.  Outside that context an eager step keeps the library's first choice and may differ in the last bits."""
    tiny = TINIES["d"]
    vocab = tiny.config["vocab_size"]
    kw = dict(max_running=24, max_seq_len=128, chunk_tokens=64, run_ahead=False)
    eager = engine(folders["d"], tiny, "bfloat16", use_graphs=False, **kw)
    graphed = engine(folders["d"], tiny, "bfloat16", use_graphs=True, **kw)
    prompts = [random_tokens(vocab, 3 + (7 * i) % 19, seed=120 + i) for i in range(24)]
    for eng in (eager, graphed):
        for i, p in enumerate(prompts):
            eng.cache.admit(i)
            eng.runner.run([StepEntry(i, p, [])])
    tokens = [random_tokens(vocab, 12, seed=200 + i) for i in range(24)]
    for step in range(12):
        live = list(range(24 - step // 4))        # 24, 23, 22 rows: one bucket, full and with padding rows
        entries = [StepEntry(i, [tokens[i][step]], [0]) for i in live]
        with eager.kernels.recurring_shapes():
            want = eager.runner.run(entries)
        got = graphed.graphs.run(entries)
        torch.cuda.synchronize()
        if len(live) == 24:      # the bucket's own number of rows: the library is asked for the same product
            assert torch.equal(got, want), (step, rel_err(got, want))
        else:                    # fewer rows run eagerly as a product of fewer rows, for which the library may choose otherwise
            assert rel_err(got, want) <= 1e-2, (step, rel_err(got, want))
    assert graphed.graphs.replays == 12 and len(graphed.graphs._made) == 1


def test_a_replayed_step_that_finds_no_page_leaves_the_books_as_they_were(folders):
    """Requests admitted without a promise (as trace replay admits them) can run out of pages in the middle of a
    step's bookkeeping: the first request of the step has been given its position, the second finds no page.  The
    step then raises with every request as long as before, and runs once a page is free."""
    from simple_inference_amd.cache.allocator import OutOfPages
    tiny = TINIES["d"]
    vocab, ps = tiny.config["vocab_size"], tiny.page_size
    eng = engine(folders["d"], tiny, "bfloat16", use_graphs=True, max_seq_len=64, num_kv_blocks=3, run_ahead=False)
    lengths = {1: ps - 1, 2: ps, 3: 5}        # request 2 fills its page exactly: its next token needs a new one
    for rid, n in lengths.items():
        eng.cache.admit(rid)
        eng.runner.run([StepEntry(rid, random_tokens(vocab, n, seed=rid), [])])
    assert eng.cache.free_pages() == 0
    entries = [StepEntry(1, [7], [0]), StepEntry(2, [8], [0])]
    with pytest.raises(OutOfPages):
        eng.graphs.run(entries)
    assert {rid: eng.cache.lengths[rid] for rid in lengths} == lengths
    eng.cache.check()
    eng.cache.release(3)                      # a page comes back: the same step now runs
    logits = eng.graphs.run(entries)
    torch.cuda.synchronize()
    assert logits.shape[0] == 2 and eng.cache.lengths[1] == ps and eng.cache.lengths[2] == ps + 1
    eager = engine(folders["d"], tiny, "bfloat16", use_graphs=False, max_seq_len=64, num_kv_blocks=3)
    for rid in (1, 2):
        eager.cache.admit(rid)
        eager.runner.run([StepEntry(rid, random_tokens(vocab, lengths[rid], seed=rid), [])])
    assert torch.equal(logits, eager.runner.run(entries))


def test_long_decoding_crosses_the_length_buckets_of_the_graphs(folders):
    """Decoding from 500 to 1,040 tokens of context: the replayed graphs change from the 512-token bucket to the
    1,024-token one and on to the last (other attention grids and key splits), and every token stays the one an
    eager engine gives (float32: greedy tokens are equal; bfloat16, where the splits show in the last bits and a
    tiny model's greedy choice hangs on them: the logits of the same given tokens stay within rounding)."""
    tiny = TINIES["d"]
    vocab = tiny.config["vocab_size"]
    prompt = random_tokens(vocab, 500, seed=140)
    kw = dict(max_seq_len=1100, max_running=2, chunk_tokens=256)
    graphed = engine(folders["d"], tiny, "float32", use_graphs=True, **kw)
    eager = engine(folders["d"], tiny, "float32", use_graphs=False, **kw)
    a = graphed.add_request(prompt, max_new_tokens=540)
    b = eager.add_request(prompt, max_new_tokens=540)
    graphed.run()
    eager.run()
    assert sorted(kv for _, kv in graphed.graphs._made) == [512, 1024, 1100]
    assert a.generated == b.generated

    graphed = engine(folders["d"], tiny, "bfloat16", use_graphs=True, **kw)
    eager = engine(folders["d"], tiny, "bfloat16", use_graphs=False, **kw)
    for eng in (graphed, eager):
        eng.cache.admit(1)
        eng.runner.run([StepEntry(1, prompt, [])])
    given = random_tokens(vocab, 540, seed=141)
    worst = 0.0
    for t in given:
        worst = max(worst, rel_err(graphed.graphs.run([StepEntry(1, [t], [0])]), eager.runner.run([StepEntry(1, [t], [0])])))
    assert sorted(kv for _, kv in graphed.graphs._made) == [512, 1024, 1100]
    assert worst <= TOLERANCE["hip-bf16"], worst   # two bfloat16 paths: no further apart than either may be from the plain one


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_logits(folders, dtype):
    tiny = TINIES["c"]
    eng = engine(folders["c"], tiny, dtype, use_graphs=True)
    prompt = random_tokens(tiny.config["vocab_size"], 50, seed=80)
    eng.cache.admit(1)
    eng.runner.run([StepEntry(1, prompt[:30], [])])
    ref = plain.forward(*plain.read_model(folders["c"]), prompt)
    for i in range(30, 50):
        logits = eng.graphs.run([StepEntry(1, [prompt[i]], [0])])
        assert rel_err(logits, ref[i:i + 1]) <= (2.5e-2 if dtype == "bfloat16" else 2e-5)


def test_temperature_sampling_on_the_gpu_follows_the_request_seed(folders):
    tiny = TINIES["a"]
    cfg, w = plain.read_model(folders["a"])
    prompts = [random_tokens(256, n, seed=90 + i) for i, n in enumerate((9, 13))]
    params = [SamplingParams(temperature=0.8, seed=7 + i, max_new_tokens=6, top_k=k, top_p=p)
              for i, (k, p) in enumerate(((0, 1.0), (12, 0.9)))]
    outs = []
    for kw in (dict(max_running=1), dict(max_running=2, chunk_tokens=4)):
        eng = engine(folders["a"], tiny, "float32", **kw)
        reqs = [eng.add_request(p, params=sp) for p, sp in zip(prompts, params)]
        eng.run()
        outs.append([r.generated for r in reqs])
    assert outs[0] == outs[1]
    for prompt, sp, got in zip(prompts, params, outs[0]):
        toks = list(prompt)
        for n, t in enumerate(got):
            logits = plain.forward(cfg, w, toks)[-1]
            assert t == plain.sample_with_uniform(logits, uniform_for(sp.seed, n), sp.temperature, sp.top_k, sp.top_p)
            toks.append(t)


@pytest.mark.parametrize("name", ["b", "c"])
def test_random_request_streams_generate_what_each_request_generates_alone(folders, name):
    """Forty requests of random lengths, with and without shared prefixes, greedy and sampled with seeds of their
    own, arrive a few per step and run through engines with few pages, small portions, graphs and prefix reuse:
    every request generates exactly the tokens it generates when it runs alone (32-bit, so that no rounding
    difference between batch shapes can flip a token).  Several engines with graphs are made and dropped in turn."""
    import random
    folder, tiny = folders[name], TINIES[name]
    V = tiny.config["vocab_size"]
    rng = random.Random(7)
    shared = [rng.randrange(V) for _ in range(60)]
    reqs = []
    for _ in range(40):
        base = shared[:rng.randint(0, len(shared))] if rng.random() < 0.5 else []
        prompt = base + [rng.randrange(V) for _ in range(rng.randint(1, 120))]
        params = SamplingParams(temperature=rng.choice([0.0, 0.0, 0.7, 1.5]), top_k=rng.choice([0, 5, 40]),
                                top_p=rng.choice([1.0, 0.9, 0.5]), seed=rng.randrange(1 << 30),
                                max_new_tokens=rng.randint(1, 40), ignore_eos=True)
        reqs.append((prompt, params))

    def run(requests, stagger, **kw):
        eng = Engine.from_folder(folder, EngineConfig(dtype="float32", max_seq_len=320, block_size=16, eos_id=-1, **kw))
        handles, pending, step = [], list(requests), 0
        while pending or eng.has_work():
            for _ in range(min(len(pending), random.Random(step).randint(0, 3) if stagger else len(pending))):
                prompt, params = pending.pop(0)
                handles.append(eng.add_request(prompt, params=params))
            eng.step()
            step += 1
        eng.cache.check()
        return [h.generated for h in handles]

    alone = [run([r], False, max_running=1, num_kv_blocks=64, use_graphs=False)[0] for r in reqs]
    for kw in (dict(max_running=6, num_kv_blocks=60, chunk_tokens=32, use_graphs=True, use_prefix_cache=True),
               dict(max_running=4, num_kv_blocks=40, chunk_tokens=16, use_graphs=True),
               dict(max_running=16, num_kv_blocks=400, chunk_tokens=512, use_graphs=False, use_prefix_cache=True)):
        got = run(reqs, True, **kw)
        assert [i for i, (a, b) in enumerate(zip(got, alone)) if a != b] == [], kw


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "d"])
def test_running_a_step_ahead_changes_no_token(folders, name, dtype):
    """Decode steps launched before the tokens of the step before are read: requests that end on an
    end-of-sequence token (found a step late), that end by count, that arrive while others decode and that wait
    for a slot all get the tokens they get without running ahead, sampled ones included, and every page comes
    back.  A request that has run past its end-of-sequence token keeps its row for one step, and a request that
    arrives while a step is running ahead joins one step later, so the rows of a step are then not the same in
    the two runs.  Decode steps do not mind (a row's result does not depend on the other rows, in either dtype);
    a step with a prompt in it does in bfloat16, where its products, the decoding rows' too, go to the BLAS
    library, which picks its method by the number of rows: there all requests arrive before the first step and
    find a slot at once, so that every later step is a decode step."""
    tiny = TINIES[name]
    vocab = tiny.config["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=80 + i) for i, n in enumerate((5, 23, 9, 31, 14, 3))]
    first_params = SamplingParams(max_new_tokens=12, temperature=1.0, seed=7)

    def stream(run_ahead, stop):
        eng = engine(folders[name], tiny, dtype, run_ahead=run_ahead, eos_id=stop,
                     max_running=4 if dtype == "float32" else 6, chunk_tokens=24 if dtype == "float32" else 96)
        params = [first_params,
                  SamplingParams(max_new_tokens=20, temperature=0.8, top_k=20, top_p=0.9, seed=3),
                  SamplingParams(max_new_tokens=7, temperature=0.0, ignore_eos=True),
                  SamplingParams(max_new_tokens=25, temperature=1.1, seed=9, ignore_eos=True),
                  SamplingParams(max_new_tokens=9, temperature=0.0),
                  SamplingParams(max_new_tokens=15, temperature=0.6, top_p=0.8, seed=5)]
        early = 3 if dtype == "float32" else 6
        reqs = [eng.add_request(p, params=q) for p, q in zip(prompts[:early], params[:early])]
        steps = 0
        while eng.has_work():
            eng.step()
            steps += 1
            if steps == 6:    # arrivals while the first three decode: one finds a slot, two wait for one
                reqs += [eng.add_request(p, params=q) for p, q in zip(prompts[early:], params[early:])]
            eng.cache.check()
        assert all(r.state is RequestState.FINISHED for r in reqs)
        assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()
        return [r.generated for r in reqs], eng.stats["steps_ahead"]

    # request 0 ends on a token of its own, in the middle of its allowance: what it generates in this arrangement
    # when no token stops it says which (in bfloat16 that need not be what it generates alone: its prompt shares
    # its first step with others, and the products of such a step depend on the step's size)
    first = stream(False, -1)[0][0]
    stop = next((t for i, t in enumerate(first) if 3 <= i < 10 and t not in first[:i]), None)
    assert stop is not None, first
    plain_way, none_ahead = stream(False, stop)
    ahead_way, some_ahead = stream(True, stop)
    assert none_ahead == 0 and some_ahead > 0
    assert plain_way == ahead_way
    assert plain_way[0][-1] == stop and 4 <= len(plain_way[0]) <= 10   # the end-of-sequence token ended request 0


@pytest.mark.parametrize("chunk_tokens", [1, 4, 5])
def test_portions_of_one_token_beside_decoders_with_graphs(folders, chunk_tokens):
    """A step budget at or below the number of slots: prompts are then fed a token or two at a time, and a step in
    which every request brings one token may hold a prompt's token that is not its last (nothing is sampled for
    it).  Such a step is not a decode step and must not go to a replayed graph; every request still generates
    what it generates alone."""
    tiny = TINIES["b"]
    vocab = tiny.config["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=160 + i) for i, n in enumerate((3, 10, 1, 7, 5, 9))]

    def run(prompts_now, **kw):
        eng = engine(folders["b"], tiny, "float32", **kw)
        handles, waiting, steps = [], list(prompts_now), 0
        while waiting or eng.has_work():
            if waiting and steps % 3 == 0:          # arrivals while others decode
                handles.append(eng.add_request(waiting.pop(0), max_new_tokens=6))
            eng.step()
            steps += 1
            assert steps < 400
        eng.cache.check()
        assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()
        return [h.generated for h in handles], eng

    alone = [run([p], max_running=1, use_graphs=False)[0][0] for p in prompts]
    got, eng = run(prompts, max_running=4, chunk_tokens=chunk_tokens, use_graphs=True)
    assert got == alone
    assert eng.stats["graph_fallbacks"] == 0 and eng.graphs is not None
    if chunk_tokens > 1:
        assert eng.graphs.replays > 0


@pytest.mark.parametrize("broken", ["capture", "replay"])
def test_a_graph_that_cannot_be_captured_or_replayed_falls_back_to_eager_steps(folders, broken, monkeypatch, capfd):
    """serving/engine.py:300-309,478-497 in kind: the failing call is made to raise from the host; the step runs
    eagerly on the same books (no page taken twice, no position skipped) and every token is what it is without
    graphs."""
    from simple_inference_amd.engine.graphs import GraphedDecode
    tiny = TINIES["d"]
    vocab = tiny.config["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=170 + i) for i, n in enumerate((9, 30, 4))]
    want = []
    for dtype in ("float32",):
        eager = engine(folders["d"], tiny, dtype, use_graphs=False)
        reqs = [eager.add_request(p, max_new_tokens=10) for p in prompts]
        eager.run()
        want = [r.generated for r in reqs]
    eng = engine(folders["d"], tiny, "float32", use_graphs=True)
    calls = {"n": 0}
    if broken == "capture":
        def fail(self, size, kv_bound):
            raise RuntimeError("no memory for the graph's private pool (made up by the test)")
        monkeypatch.setattr(GraphedDecode, "capture", fail)
    else:
        real = GraphedDecode.capture

        def capture_then_break(self, size, kv_bound):
            bucket = real(self, size, kv_bound)

            class Broken:
                def replay(_):
                    calls["n"] += 1
                    if calls["n"] == 3:
                        raise RuntimeError("replay refused (made up by the test)")
                    bucket_graph.replay()
            bucket_graph = bucket.graph
            bucket.graph = Broken()
            return bucket
        monkeypatch.setattr(GraphedDecode, "capture", capture_then_break)
    reqs = [eng.add_request(p, max_new_tokens=10) for p in prompts]
    eng.run()
    assert [r.generated for r in reqs] == want
    assert eng.graphs is None and eng.stats["graph_fallbacks"] == 1
    assert "decode steps run eagerly from here on" in capfd.readouterr().err
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()


@pytest.mark.parametrize("name", ["a", "d"])
def test_decode_steps_in_bfloat16_do_not_depend_on_the_batch(folders, name):
    """serving/test_engine.py:151-190 in the serving dtype.  Each request's prompt is run the same way in every
    arrangement (alone, whole); then it decodes given tokens alone, among three others, among fifteen others, and
    in replayed graphs padded to their bucket under a larger bound on the length: its logits are the same bit for
    bit, because neither the few-row products nor the split of its keys between workgroups look at the rest of
    the batch.  (A step of more than 16 rows sends its products to the BLAS library, which chooses its method by
    the number of rows: such steps agree within rounding, see the test below.)"""
    tiny = TINIES[name]
    vocab = tiny.config["vocab_size"]
    lengths = (5, 70, 33, 130, 1, 64, 17, 90, 12, 47, 8, 100, 3, 29, 55, 21)
    prompts = [random_tokens(vocab, n, seed=180 + i) for i, n in enumerate(lengths)]
    given = [random_tokens(vocab, 12, seed=220 + i) for i in range(len(prompts))]

    def decode(groups, graphs):
        """Logits [request][step] when the requests decode in the given groups (one batch a group and step)."""
        eng = engine(folders[name], tiny, "bfloat16", use_graphs=graphs, max_running=16, max_seq_len=1024)
        for i, p in enumerate(prompts):
            eng.cache.admit(i)
            eng.runner.run([StepEntry(i, p, [])])
        out = {i: [] for i in range(len(prompts))}
        for step in range(12):
            for group in groups:
                entries = [StepEntry(i, [given[i][step]], [0]) for i in group]
                logits = eng.graphs.run(entries) if graphs else eng.runner.run(entries)
                for row, i in enumerate(group):
                    out[i].append(logits[row].clone())
        return out

    everyone = list(range(16))
    alone = decode([[i] for i in everyone], graphs=False)
    for groups, graphs in (([everyone[:4], everyone[4:7], everyone[7:]], False), ([everyone], False),
                           ([everyone[:3], everyone[3:]], True), ([everyone[::-1]], True)):
        got = decode(groups, graphs)
        for i in everyone:
            for step in range(12):
                assert torch.equal(got[i][step], alone[i][step]), (groups, graphs, i, step)


def test_random_request_streams_in_bfloat16_stay_within_rounding_of_the_plain_implementation(folders):
    """The stream of the 32-bit test above in the serving dtype, greedy only.  Prompts are cut and batched as the
    stream has it, so a request's steps differ from its steps alone in the number of rows of their products (the
    BLAS library's choice from 17 rows on): its tokens need not be bit-equal to a solo run's, but every one of
    them must be the plain implementation's choice, or tie with it within bfloat16 rounding."""
    import random
    folder, tiny = folders["b"], TINIES["b"]
    V = tiny.config["vocab_size"]
    rng = random.Random(11)
    shared = [rng.randrange(V) for _ in range(40)]
    reqs = []
    for _ in range(14):
        base = shared[:rng.randint(0, len(shared))] if rng.random() < 0.5 else []
        reqs.append((base + [rng.randrange(V) for _ in range(rng.randint(1, 90))], rng.randint(1, 12)))
    for kw in (dict(max_running=6, num_kv_blocks=60, chunk_tokens=32, use_graphs=True, use_prefix_cache=True),
               dict(max_running=3, num_kv_blocks=40, chunk_tokens=16, use_graphs=True)):
        eng = Engine.from_folder(folder, EngineConfig(dtype="bfloat16", max_seq_len=320, block_size=16, eos_id=-1, **kw))
        handles, pending, step = [], list(reqs), 0
        while pending or eng.has_work():
            for _ in range(min(len(pending), random.Random(step).randint(0, 3))):
                prompt, n = pending.pop(0)
                handles.append(eng.add_request(prompt, max_new_tokens=n))
            eng.step()
            step += 1
        eng.cache.check()
        for (prompt, n), h in zip(reqs, handles):
            assert len(h.generated) == n
            greedy_matches_plain(folder, prompt, h.generated, "bfloat16")
