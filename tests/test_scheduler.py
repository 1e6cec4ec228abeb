"""The scheduler's decisions and the engine around it, on the CPU with the torch twins of the kernels."""

import random

import pytest

import plain_llama as plain
from helpers import TINIES, random_tokens, write_tiny_model
from simple_inference_amd import Engine, EngineConfig, RequestState, SamplingParams
from simple_inference_amd.engine import Request, Scheduler
from simple_inference_amd.sampling import uniform_for, uniforms_for
from twins import TwinKernels


def req(n_prompt, max_new=4):
    return Request(list(range(1, n_prompt + 1)), SamplingParams(max_new_tokens=max_new))


def ids(plan):
    return [(r.id, n) for r, n in plan]


def ran(plan):
    """What the engine does with a plan, as far as the scheduler can see it: the requests take their tokens."""
    for r, n in plan:
        _, samples, _ = r.take(n)
        if samples:
            r.sampled(0)


# ---- the scheduler alone ---------------------------------------------------------------------
def test_coming_in_is_first_come_first_served_without_overtaking():
    s = Scheduler(max_running=4, token_budget=1000, chunk_tokens=8)
    a, b, c = req(5), req(50), req(2)
    for r in (a, b, c):
        s.submit(r)
    fits = lambda r: r.prompt_len < 10          # b cannot get its pages
    assert s.let_in(fits) is a
    assert [r.state for r in (a, b, c)] == [RequestState.PREFILL, RequestState.WAITING, RequestState.WAITING]
    assert s.let_in(fits) is None                # c does not jump over b
    assert s.let_in() is b and s.let_in() is c and s.let_in() is None
    assert s.live == [a, b, c] and not s.queue


def test_token_budget_and_slots():
    s = Scheduler(max_running=2, token_budget=10, chunk_tokens=8)
    a, b, c = req(30), req(4), req(4)
    for r in (a, b, c):
        s.submit(r)
    assert s.let_in() is a                       # an empty engine takes any one request, however long
    assert s.let_in() is None                    # 30 + 4 > 10
    a.state = RequestState.FINISHED
    assert s.retire() == [a] and s.retire() == []
    assert s.let_in() is b and s.let_in() is c and s.let_in() is None   # two slots
    with pytest.raises(ValueError):
        s.submit(b)                              # only a waiting request can be queued


def test_the_budget_counts_tokens_in_flight():
    s = Scheduler(max_running=3, token_budget=12, chunk_tokens=8)
    a, b, c = req(5, max_new=8), req(6), req(1)
    s.submit(a), s.submit(b), s.submit(c)
    plan = s.plan()
    assert ids(plan) == [(a.id, 5), (b.id, 3)] and c.state is RequestState.WAITING   # 5 + 6 + 1 = 12 would fit, but
    ran(plan)                                                                       # the step's room was used up
    assert a.context_len == 6                    # its sampled token is in flight and counts
    assert s.let_in() is None                    # 6 + 6 + 1 > 12
    a.state = RequestState.FINISHED
    s.retire()
    assert s.let_in() is c


def test_plan_gives_decoders_one_token_then_prompt_portions_in_order():
    s = Scheduler(max_running=4, token_budget=1000, chunk_tokens=8)
    d1, d2, p1, p2 = req(3), req(3), req(20), req(5)
    for r in (d1, p1, d2, p2):
        s.submit(r)
    while s.let_in():
        pass
    ran([(d1, 3), (d2, 3), (p1, 16)])
    plan = s.plan(admit=False)
    assert ids(plan) == [(d1.id, 1), (d2.id, 1), (p1.id, 4), (p2.id, 2)]
    ran(plan)
    assert p1.state is RequestState.DECODE and p2.num_computed == 2
    assert ids(s.plan(admit=False)) == [(d1.id, 1), (p1.id, 1), (d2.id, 1), (p2.id, 3)]


def test_plan_lets_newcomers_in_only_where_there_is_room_for_their_first_tokens():
    s = Scheduler(max_running=4, token_budget=1000, chunk_tokens=8)
    a, b, c, d = req(11), req(3), req(6), req(2)
    for r in (a, b, c, d):
        s.submit(r)
    plan = s.plan()
    assert ids(plan) == [(a.id, 8)]                              # a fills the step: nobody else enters yet
    assert [r.state for r in (a, b, c)] == [RequestState.PREFILL, RequestState.WAITING, RequestState.WAITING]
    ran(plan)
    plan = s.plan()                                              # a's rest, all of b, the start of c
    assert ids(plan) == [(a.id, 3), (b.id, 3), (c.id, 2)]
    assert d.state is RequestState.WAITING and len(s.live) == 3
    ran(plan)
    ran([(c, 4)])
    # the gate still decides, and nobody overtakes the head of the queue
    assert ids(s.plan(lambda r: False)) == [(a.id, 1), (b.id, 1), (c.id, 1)]
    assert ids(s.plan(admit=False)) == [(a.id, 1), (b.id, 1), (c.id, 1)]
    assert ids(s.plan(lambda r: True)) == [(a.id, 1), (b.id, 1), (c.id, 1), (d.id, 2)]


def test_a_request_keeps_its_own_books():
    r = req(5, max_new=2)
    assert r.tokens_wanted(8) == 0 and r.total_len == 7      # waiting: it brings nothing
    r.enter(slot=3, reused_tokens=2)
    assert (r.state, r.slot, r.num_computed, r.cached_prefix_len) == (RequestState.PREFILL, 3, 2, 2)
    assert r.tokens_wanted(2) == 2 and r.tokens_wanted(99) == 3
    assert r.take(2) == ([3, 4], False, None)
    with pytest.raises(ValueError):
        r.take(2)                                            # one token is left
    assert r.take(1) == ([5], True, None)
    r.sampled(row=4)
    assert r.state is RequestState.DECODE and r.context_len == 6 and r.length_is_certain_after_next_token()
    assert r.take(1) == ([0], True, 4)                       # its input is still on the device, in row 4
    r.sampled(row=0)
    assert not r.length_is_certain_after_next_token()
    assert r.deliver(9) and r.generated == [9] and r.state is RequestState.DECODE
    assert r.deliver(2, eos_ids=(2,)) and r.eos_hit and r.state is RequestState.FINISHED and r.slot is None
    r.in_flight = 1
    assert not r.deliver(11) and r.generated == [9, 2]       # sampled a step too far: dropped
    q = req(1, max_new=1)
    q.enter(0)
    q.take(1), q.sampled(0)
    assert q.deliver(2, eos_ids=()) and q.finish_reason == "length"
    with pytest.raises(ValueError):
        req(3).take(1)                                       # not admitted
    # an end by count is known before the last token is read: the request ends ahead and takes part in nothing more
    e = req(2, max_new=2)
    e.enter(1)
    e.take(2), e.sampled(0)
    assert not e.last_token_is_in_flight()
    with pytest.raises(ValueError):
        e.end_ahead()                                        # one more token may follow
    assert e.deliver(5)
    e.take(1), e.sampled(3)
    assert e.last_token_is_in_flight()
    e.end_ahead()
    assert e.state is RequestState.ENDING and e.slot is None and e.tokens_wanted(8) == 0
    assert e.deliver(7) and e.generated == [5, 7] and e.state is RequestState.FINISHED and e.finish_reason == "length"
    s = Scheduler(max_running=2, token_budget=100, chunk_tokens=8)
    a, b = req(3, max_new=1), req(3, max_new=4)
    s.submit(a), s.submit(b)
    assert ids(s.plan(lambda r: True)) == [(a.id, 3), (b.id, 3)]
    for r in (a, b):
        r.take(3), r.sampled(0)
    a.end_ahead()
    assert s.retire() == [a] and ids(s.plan()) == [(b.id, 1)]  # gone from the running before its token is read


# ---- the engine on the CPU -----------------------------------------------------------------------
@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return write_tiny_model(tmp_path_factory.mktemp("sched"), TINIES["b"], seed=21)


def engine(folder, **kw):
    base = dict(device="cpu", dtype="float32", max_seq_len=128, block_size=8, max_running=4, chunk_tokens=16,
                eos_id=-1)
    base.update(kw)
    return Engine.from_folder(folder, EngineConfig(**base), TwinKernels())


def plain_greedy(folder, prompt, n):
    cfg, w = plain.read_model(folder)
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]


PROMPTS = [random_tokens(384, n, seed=40 + i) for i, n in enumerate((1, 17, 40, 70))]


def test_tokens_do_not_depend_on_batching_queueing_or_portions(folder):
    want = [plain_greedy(folder, p, 6) for p in PROMPTS]
    for kw in (dict(max_running=1), dict(max_running=4), dict(max_running=2), dict(max_running=4, chunk_tokens=5),
               dict(max_running=3, num_kv_blocks=24, chunk_tokens=64)):
        eng = engine(folder, **kw)
        reqs = [eng.add_request(p, max_new_tokens=6) for p in PROMPTS]
        eng.run()
        assert [r.generated for r in reqs] == want, kw
        assert all(r.state is RequestState.FINISHED and r.slot is None for r in reqs)
        assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks() and eng.cache.slots.free_slots == kw["max_running"]
        eng.cache.check()


@pytest.mark.parametrize("run_ahead", [False, True])
def test_a_request_that_finds_no_pages_waits_for_a_finished_one(folder, run_ahead):
    """serving/test_paged_kv_cache.py:247-269: 2 pages, two 3-token prompts with 1 new token each.  Running ahead,
    the engine knows that the first request's one token is its last before it has read it: the second request gets
    the page in the same call, and its step is on its way when the call returns."""
    eng = engine(folder, block_size=4, num_kv_blocks=1, max_running=2, run_ahead=run_ahead)
    a = eng.add_request([1, 4, 6], max_new_tokens=1)
    b = eng.add_request([1, 5, 9], max_new_tokens=1)
    eng.step()
    assert a.state is RequestState.FINISHED and a.slot is None
    if run_ahead:
        assert b.state is RequestState.DECODE and b.num_computed == 3 and b.in_flight == 1
    else:
        assert b.state is RequestState.WAITING
    eng.step()
    assert b.state is RequestState.FINISHED and eng.cache.free_pages() == 1
    assert a.generated == plain_greedy(folder, [1, 4, 6], 1) and b.generated == plain_greedy(folder, [1, 5, 9], 1)


def test_first_token_comes_from_the_step_that_ends_the_prompt(folder):
    eng = engine(folder, chunk_tokens=16, run_ahead=False)   # the request's books are looked at between the steps
    r = eng.add_request(PROMPTS[2], max_new_tokens=3)       # 40 tokens: portions 16, 16, 8
    emitted = [eng.step() for _ in range(3)]
    assert emitted[0] == {} and emitted[1] == {} and list(emitted[2]) == [r.id]
    assert r.state is RequestState.DECODE and r.num_computed == 40
    eng.step()
    assert r.num_generated == 2 and r.num_computed == 41


def test_decoders_go_on_while_a_long_prompt_is_fed_in_portions(folder):
    eng = engine(folder, chunk_tokens=9)
    short = eng.add_request(PROMPTS[0], max_new_tokens=8)
    eng.step()
    long = eng.add_request(PROMPTS[3], max_new_tokens=2)     # 70 tokens at 8 a step beside the decoder
    for _ in range(4):
        out = eng.step()
        assert short.id in out and long.id not in out
    eng.run()
    assert short.generated == plain_greedy(folder, PROMPTS[0], 8)
    assert long.generated == plain_greedy(folder, PROMPTS[3], 2)


def test_temperature_sampling_is_seeded_per_request_and_independent_of_the_batch(folder):
    cfg, w = plain.read_model(folder)
    params = [SamplingParams(temperature=0.8, seed=100 + i, max_new_tokens=6, top_k=k, top_p=p)
              for i, (k, p) in enumerate(((0, 1.0), (5, 1.0), (0, 0.7), (20, 0.9)))]
    want = []
    for prompt, sp in zip(PROMPTS, params):
        toks = list(prompt)
        for n in range(6):
            logits = plain.forward(cfg, w, toks)[-1]
            toks.append(plain.sample_with_uniform(logits, uniform_for(sp.seed, n), sp.temperature, sp.top_k, sp.top_p))
        want.append(toks[len(prompt):])
    for kw in (dict(max_running=1), dict(max_running=4, chunk_tokens=7)):
        eng = engine(folder, **kw)
        reqs = [eng.add_request(p, params=sp) for p, sp in zip(PROMPTS, params)]
        eng.run()
        assert [r.generated for r in reqs] == want, kw
    assert len({tuple(t) for t in want}) == 4


def test_a_batch_of_uniform_numbers_is_the_numbers_one_by_one():
    """The sampler computes a step's uniform numbers for all its rows at once: bit for bit what ``uniform_for`` gives
    for each (seed, draw), also for seeds that are negative or wider than 64 bits, and all in [0, 1)."""
    rng = random.Random(5)
    seeds = [0, 1, -1, -12345, 2 ** 63, 2 ** 64 - 1, 2 ** 64, 2 ** 70 + 3] + [rng.getrandbits(64) for _ in range(100)]
    draws = [0, 1, 2, 2 ** 31, 2 ** 63, 7, 10 ** 6, 3] + [rng.randrange(10 ** 6) for _ in range(100)]
    batch = uniforms_for(seeds, draws)
    assert batch.dtype.name == "float32" and batch.shape == (len(seeds),)
    assert [float(u) for u in batch] == [uniform_for(s, n) for s, n in zip(seeds, draws)]
    assert all(0.0 <= float(u) < 1.0 for u in batch)


def test_stops_at_eos_and_generate_does_not_yield_it(folder):
    first = plain_greedy(folder, PROMPTS[1], 3)
    eng = engine(folder, eos_id=first[2])
    r = eng.add_request(PROMPTS[1], max_new_tokens=10)
    eng.run()
    assert r.generated == first and r.eos_hit                 # EOS is kept in generated (serving/engine.py:449-460)
    eng = engine(folder, eos_id=first[2])
    assert list(eng.generate(PROMPTS[1], max_new_tokens=10, temperature=0.0)) == first[:2]
    ignoring = engine(folder, eos_id=first[2])
    r = ignoring.add_request(PROMPTS[1], params=SamplingParams(max_new_tokens=5, ignore_eos=True))
    ignoring.run()
    assert r.num_generated == 5


def test_add_request_checks(folder):
    eng = engine(folder, max_seq_len=32, num_kv_blocks=2)
    for prompt, new, word in (([], 1, "empty"), ([1, 2], 0, "max_new_tokens"), ([1] * 30, 3, "max_seq_len"),
                              ([1] * 10, 10, "more pages"), ([1, 999], 2, "out-of-range")):
        with pytest.raises(ValueError, match=word):
            eng.add_request(prompt, max_new_tokens=new)


def test_reset_gives_everything_back(folder):
    eng = engine(folder)
    for p in PROMPTS:
        eng.add_request(p, max_new_tokens=4)
    eng.step()
    eng.reset()
    assert not eng.has_work() and eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()
    r = eng.add_request(PROMPTS[1], max_new_tokens=2)
    eng.run()
    assert r.generated == plain_greedy(folder, PROMPTS[1], 2)


def test_generate_with_stats_has_the_reference_names(folder):
    eng = engine(folder)
    tokens, stats = eng.generate_with_stats(PROMPTS[1], max_new_tokens=4, temperature=0.0)
    assert tokens == plain_greedy(folder, PROMPTS[1], 4)
    for key in ("ttft_ms", "tpot_ms", "prefill_ms", "decode_tok_s", "total_wall_ms", "total_tok_s", "peak_vram_gb",
                "prompt_tokens", "new_tokens"):
        assert key in stats


def test_running_ahead_books_the_same_tokens_and_pages(folder):
    """The engine's bookkeeping when steps are launched before the tokens of the step before are read (decoded
    tokens and prompt portions alike; the token ids then come from the sampler's output, here a CPU tensor): a
    request that ends on an end-of-sequence token (it has then run one token too far), ends by count, arrivals
    that find a slot or wait for one.  Tokens, states and pages are those of an engine that never runs ahead."""
    first = plain_greedy(folder, PROMPTS[1], 12)
    stop = next(t for i, t in enumerate(first) if i >= 3 and t not in first[:i])

    def stream(run_ahead):
        eng = engine(folder, eos_id=stop, run_ahead=run_ahead, max_running=3)
        params = [SamplingParams(max_new_tokens=12), SamplingParams(max_new_tokens=9, temperature=0.9, seed=4, ignore_eos=True),
                  SamplingParams(max_new_tokens=20, ignore_eos=True), SamplingParams(max_new_tokens=6, temperature=1.2, top_k=30, seed=8),
                  SamplingParams(max_new_tokens=15, ignore_eos=True)]
        prompts = [PROMPTS[1], PROMPTS[0], PROMPTS[2], PROMPTS[1][:9], PROMPTS[3][:30]]
        reqs = [eng.add_request(p, params=q) for p, q in zip(prompts[:2], params[:2])]
        emitted_by_step = []
        while eng.has_work():
            emitted_by_step.append(eng.step())
            if len(emitted_by_step) == 5:
                reqs += [eng.add_request(p, params=q) for p, q in zip(prompts[2:], params[2:])]
            eng.cache.check()
        assert all(r.state is RequestState.FINISHED for r in reqs)
        assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()
        # every token was reported by exactly one step, in order
        for r in reqs:
            assert [e[r.id] for e in emitted_by_step if r.id in e] == r.generated
        return [r.generated for r in reqs], eng.stats["steps_ahead"]

    plain_way, none_ahead = stream(False)
    ahead_way, some_ahead = stream(True)
    assert none_ahead == 0 and some_ahead > 5
    assert ahead_way == plain_way
    assert plain_way[0] == first[:first.index(stop) + 1]          # ended on the end-of-sequence token
    assert len(plain_way[2]) == 20 and len(plain_way[4]) == 15     # ended by count


@pytest.mark.parametrize("chunk_tokens", [1, 4])
def test_a_step_budget_at_or_below_the_slots_feeds_prompts_token_by_token(folder, chunk_tokens):
    want = [plain_greedy(folder, p, 5) for p in PROMPTS[:3]]
    eng = engine(folder, max_running=4, chunk_tokens=chunk_tokens)
    reqs = [eng.add_request(p, max_new_tokens=5) for p in PROMPTS[:3]]
    steps = 0
    while eng.has_work():
        eng.step()
        steps += 1
        assert steps < 500
    assert [r.generated for r in reqs] == want
    eng.cache.check()


def test_named_ranges_wrap_the_phases_of_a_step(folder):
    eng = engine(folder, profile_ranges=True)
    eng.add_request(PROMPTS[1], max_new_tokens=2)
    eng.run()
    names = eng.ranges.entered
    assert names[:2] == ["engine.schedule", "engine.forward"]
    assert all(names[i - 1] == "engine.forward" for i, n in enumerate(names) if n == "engine.sample")
    assert {"engine.schedule", "engine.forward", "engine.sample", "engine.collect"} <= set(names)
    off = engine(folder)
    off.add_request(PROMPTS[1], max_new_tokens=2)
    off.run()
    assert off.ranges.entered == []


def test_the_engine_goes_on_eagerly_when_its_graphs_give_up(folder, capsys):
    """The engine's side of the fallback, with a stand-in for the graphs (the real ones need a GPU): a stand-in
    that books a step as the real one does, then fails and takes its booking back."""
    from simple_inference_amd.engine.graphs import GraphUnavailable

    class GraphsThatFail:
        def __init__(self, eng, after):
            self.eng, self.after, self.calls = eng, after, 0

        def can_run(self, entries):
            return all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)

        def run(self, entries, device_tokens=None):
            self.calls += 1
            if self.calls <= self.after:
                return self.eng.runner.run(entries, device_tokens)
            for e in entries:
                self.eng.cache.extend(e.req, 1)
            for e in entries:
                self.eng.cache.retract(e.req, 1)
            raise GraphUnavailable("made up by the test") from RuntimeError("replay refused")

    want = [plain_greedy(folder, p, 6) for p in PROMPTS[:3]]
    eng = engine(folder, max_running=4)
    eng.graphs = GraphsThatFail(eng, after=2)
    reqs = [eng.add_request(p, max_new_tokens=6) for p in PROMPTS[:3]]
    eng.run()
    assert [r.generated for r in reqs] == want
    assert eng.graphs is None and eng.stats["graph_fallbacks"] == 1
    assert "replay refused" in capsys.readouterr().err
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cfg.resolved_num_kv_blocks()


def test_generate_takes_text_where_the_folder_has_a_tokenizer(tmp_path):
    """Reference: ``generate.py:50-119`` takes the prompt as text and yields pieces of text.  The same request given
    as token ids yields the ids those pieces decode from."""
    from tokenizers import Tokenizer as Fast
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    folder = write_tiny_model(tmp_path, TINIES["a"], seed=11)
    words = {f"w{i}": i for i in range(256)}
    fast = Fast(WordLevel(words, unk_token="w0"))
    fast.pre_tokenizer = Whitespace()
    fast.save(str(tmp_path / "tokenizer.json"))
    eng = engine(folder, block_size=4)
    text = "w17 w5 w200 w33"
    ids = [TINIES["a"].config["bos_token_id"], 17, 5, 200, 33]
    assert eng.tokenizer().encode(text) == ids
    by_ids = list(eng.generate(ids, max_new_tokens=6, temperature=0.0))
    pieces = list(eng.generate(text, max_new_tokens=6, temperature=0.0))
    assert "".join(pieces) == eng.tokenizer().decode(by_ids) and len(pieces) == len(by_ids)
    out, stats = eng.generate_with_stats(text, max_new_tokens=6, temperature=0.0)
    assert out == "".join(pieces) and stats["prompt_tokens"] == 5
    other = Engine.from_random(TINIES["a"].config, 0, EngineConfig(device="cpu", dtype="float32", max_seq_len=64,
                                                                  use_graphs=False), TwinKernels())
    with pytest.raises(ValueError, match="token ids"):
        next(other.generate("w1 w2"))
