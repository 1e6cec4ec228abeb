"""The step function against the plain implementation, under every way of cutting the work.

The same tests run on the CPU with the torch twins of the kernels (marked not gpu: they
test the cache manager and the batch layout) and on the GPU with the HIP kernels in float32
and in bfloat16 (marked gpu).
"""

import pytest
import torch

from helpers import TINIES, TOLERANCE, make_runner, plain_logits, random_tokens, rel_err, write_tiny_model
from simple_inference_amd.engine import StepEntry

BACKENDS = [
    pytest.param("twins"),
    pytest.param("hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip-bf16", marks=pytest.mark.gpu),
]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, tiny in TINIES.items():
        out[name] = write_tiny_model(tmp_path_factory.mktemp(f"tiny_{name}"), tiny, seed=11 + len(name))
    return out


def replay(runner, cache, schedule):
    """schedule: list of steps; a step is (entries, ends); an entry is (req, tokens, want).
    Returns {req: {position: logits row}}."""
    got = {}
    fed = {}
    for entries, ends in schedule:
        step_entries = []
        for req, tokens, want in entries:
            if req not in cache.lengths:
                cache.admit(req)
                fed[req] = 0
            step_entries.append(StepEntry(req, tokens, want))
        logits = runner.run(step_entries)
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


def check_against_plain(got, prompts, folder, backend):
    worst = 0.0
    for req, rows in got.items():
        ref = plain_logits(folder, prompts[req])
        pos = sorted(rows)
        mine = torch.stack([rows[p] for p in pos])
        worst = max(worst, rel_err(mine, ref[pos]))
    assert worst <= TOLERANCE[backend], f"worst relative difference {worst:.3e} > {TOLERANCE[backend]:.1e}"
    return worst


def cut(tokens, sizes):
    """Cuts a token list into portions whose sizes cycle through ``sizes``."""
    out, i, k = [], 0, 0
    while i < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - i)
        out.append(tokens[i:i + n])
        i += n
        k += 1
    return out


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(TINIES))
def test_whole_prompts_alone(folders, backend, name):
    tiny = TINIES[name]
    runner, cache, mcfg = make_runner(folders[name], backend, tiny.page_size, num_pages=64)
    prompts = {i: random_tokens(mcfg.vocab_size, n, seed=i) for i, n in enumerate((1, 5, 17, 70, 131))}
    schedule = [([(r, t, list(range(len(t))))], [r]) for r, t in prompts.items()]
    got = replay(runner, cache, schedule)
    check_against_plain(got, prompts, folders[name], backend)
    assert all(cache.free_pages(g) == 64 for g in range(len(cache.groups)))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(TINIES))
def test_last_32_tokens_one_by_one(folders, backend, name):
    tiny = TINIES[name]
    runner, cache, mcfg = make_runner(folders[name], backend, tiny.page_size, num_pages=64)
    tokens = random_tokens(mcfg.vocab_size, 97, seed=5)
    head = len(tokens) - 32
    schedule = [([(0, tokens[:head], [head - 1])], [])]
    schedule += [([(0, [tokens[i]], [0])], []) for i in range(head, len(tokens))]
    got = replay(runner, cache, schedule)
    assert sorted(got[0]) == list(range(head - 1, len(tokens)))
    check_against_plain(got, {0: tokens}, folders[name], backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(TINIES))
def test_portions_of_changing_size(folders, backend, name):
    tiny = TINIES[name]
    runner, cache, mcfg = make_runner(folders[name], backend, tiny.page_size, num_pages=64)
    tokens = random_tokens(mcfg.vocab_size, 150, seed=6)
    schedule = [([(0, part, list(range(len(part))))], []) for part in cut(tokens, [2, 7, 3, 16, 2, 33, 5, 64, 9])]
    got = replay(runner, cache, schedule)
    check_against_plain(got, {0: tokens}, folders[name], backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(TINIES))
def test_mixed_requests_with_page_reuse(folders, backend, name):
    """Up to four live requests; portions of some beside single tokens of others; the pool is so
    small that pages of finished requests are handed out again."""
    tiny = TINIES[name]
    ps = tiny.page_size
    lengths = [70, 45, 90, 33, 64, 51, 80]
    vocab = tiny.config["vocab_size"]
    prompts = {i: random_tokens(vocab, n, seed=100 + i) for i, n in enumerate(lengths)}
    # four largest live at once, each rounded up to whole pages
    pool = sum(sorted(-(-n // ps) for n in lengths)[-4:])
    runner, cache, mcfg = make_runner(folders[name], backend, ps, num_pages=pool)

    # every request: a first portion, then portions of changing size, its last 6 tokens one by one
    plans = {}
    for r, toks in prompts.items():
        body, tail = toks[:-6], toks[-6:]
        plans[r] = cut(body, [11 + r, 2, 5, 23]) + [[t] for t in tail]
    waiting = list(prompts)
    live, schedule, pages_seen = [], [], set()
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for r in list(live):
            if (len(schedule) + r) % 5 == 4 and len(live) > 1:
                continue  # a request may be left out of a step and go on later
            part = plans[r].pop(0)
            entries.append((r, part, list(range(len(part)))))
            if not plans[r]:
                ends.append(r)
                live.remove(r)
        schedule.append((entries, ends))
    assert any(len(e) == 4 for e, _ in schedule)
    got = replay(runner, cache, schedule)
    check_against_plain(got, prompts, folders[name], backend)
    assert all(cache.free_pages(g) == pool for g in range(len(cache.groups)))


@pytest.mark.parametrize("backend", BACKENDS)
def test_first_tokens_of_a_sequence(folders, backend):
    """Position 0 sees one key; its logits are those of a one-token sequence."""
    tiny = TINIES["b"]
    runner, cache, mcfg = make_runner(folders["b"], backend, tiny.page_size, num_pages=16)
    tokens = random_tokens(mcfg.vocab_size, 3, seed=9)
    got = replay(runner, cache, [([(0, [tokens[0]], [0])], []), ([(0, [tokens[1]], [0])], []),
                                 ([(0, [tokens[2]], [0])], [0])])
    check_against_plain(got, {0: tokens}, folders["b"], backend)
    one = plain_logits(folders["b"], tokens[:1])
    assert rel_err(got[0][0][None], one) <= TOLERANCE[backend]


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(folders, backend):
    tiny = TINIES["a"]
    runner, cache, mcfg = make_runner(folders["a"], backend, tiny.page_size, num_pages=128)
    tokens = random_tokens(mcfg.vocab_size, 300, seed=10)
    schedule = [([(0, tokens[:4], [3])], [])] + [([(0, [t], [0])], []) for t in tokens[4:]]
    got = replay(runner, cache, schedule)
    check_against_plain(got, {0: tokens}, folders["a"], backend)


@pytest.mark.gpu
def test_float32_stored_weights_in_the_bfloat16_engine(tmp_path):
    """A tensor stored in 32 bit stays so: its products run in float32 between bfloat16 activations."""
    tiny = TINIES["a"]
    folder = write_tiny_model(tmp_path, tiny, seed=4, storage="float32")
    runner, cache, mcfg = make_runner(folder, "hip-bf16", tiny.page_size, num_pages=64)
    assert runner.model.embedding.weight.dtype == torch.float32
    assert runner.model.layers[0].mixer.w_qkv.dtype == torch.float32
    tokens = random_tokens(mcfg.vocab_size, 40, seed=3)
    got = replay(runner, cache, [([(0, tokens[:33], list(range(33)))], []), ([(0, tokens[33:], list(range(7)))], [0])])
    check_against_plain(got, {0: tokens}, folder, "hip-bf16")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "d"])
def test_a_block_in_one_call_is_the_block_part_by_part(folders, name):
    """Steps of many tokens make a block's launches in one native call; the launches are the parts' own, so logits
    and cache are the same bit for bit as part by part: prompt portions of changing size beside decoded tokens of
    another request, whose pages are used again by a third."""
    tiny = TINIES[name]
    outs = []
    for whole in (True, False):
        runner, cache, mcfg = make_runner(folders[name], "hip-bf16", tiny.page_size, num_pages=-(-250 // tiny.page_size))
        runner.kernels.whole_blocks = whole
        a, b, c = (random_tokens(mcfg.vocab_size, n, seed=20 + i) for i, n in enumerate((150, 60, 90)))
        schedule = [([(0, a[:70], [69]), (1, b[:30], [3, 29])], []),
                    ([(1, [b[30]], [0]), (0, a[70:131], [0, 60])], []),
                    ([(0, a[131:], [18]), (1, b[31:], list(range(29)))], [1]),
                    ([(2, c[:64], [63]), (0, [a[-1]], [])], [0]),
                    ([(2, c[64:], [25])], [2])]
        got = replay(runner, cache, schedule)
        outs.append((got, [g.k.clone() for g in cache.groups], [g.v.clone() for g in cache.groups]))
        runner.kernels.whole_blocks = True
    (got_whole, k_whole, v_whole), (got_parts, k_parts, v_parts) = outs
    assert got_whole.keys() == got_parts.keys()
    for req in got_whole:
        assert got_whole[req].keys() == got_parts[req].keys()
        for pos in got_whole[req]:
            assert torch.equal(got_whole[req][pos], got_parts[req][pos]), (req, pos)
    for x, y in zip(k_whole + v_whole, k_parts + v_parts):
        assert torch.equal(x, y)


@pytest.mark.gpu
def test_few_token_steps_take_the_products_with_fused_epilogues(folders):
    """Configuration D has the sizes for them: a step of few tokens in bfloat16 runs one product that rotates and
    writes the cache and two that add into the residual per layer, and no rotation or norm kernel between layers;
    a step of many tokens runs none of them: its launches are made by one call a layer, or part by part.  (That their logits agree with the plain implementation is what the
    other tests of this file check, for D as for the others.)"""
    tiny = TINIES["d"]
    runner, cache, mcfg = make_runner(folders["d"], "hip-bf16", tiny.page_size, num_pages=64)
    core = runner.kernels.core
    counted = ("sia_gemm_skinny_rope", "sia_gemm_skinny_residual", "sia_gemm_skinny_residual_tiled",
               "sia_gemm_skinny_swiglu", "sia_rope_kv_write", "sia_add_rmsnorm", "sia_prenorm_block")
    calls = {name: 0 for name in counted}
    real = {name: getattr(core, name) for name in counted}

    def counting(name):
        def call(*args):
            calls[name] += 1
            return real[name](*args)
        return call

    for name in counted:
        setattr(core, name, counting(name))
    try:
        layers = mcfg.num_hidden_layers
        tokens = random_tokens(mcfg.vocab_size, 40, seed=5)
        cache.admit("r")
        runner.run([StepEntry("r", tokens[:20], [19])])       # many tokens: the library's products, separate kernels,
        assert calls["sia_gemm_skinny_rope"] == calls["sia_gemm_skinny_residual"] == 0    # launched by one call a layer
        assert calls["sia_gemm_skinny_residual_tiled"] == 0
        assert calls["sia_prenorm_block"] == layers and calls["sia_rope_kv_write"] == 0 and calls["sia_add_rmsnorm"] == 1
        for name in counted:
            calls[name] = 0
        runner.kernels.whole_blocks = False                    # the same launches part by part
        runner.run([StepEntry("r", tokens[20:37], [16])])
        runner.kernels.whole_blocks = True
        assert calls["sia_gemm_skinny_rope"] == calls["sia_gemm_skinny_residual"] == calls["sia_prenorm_block"] == 0
        assert calls["sia_gemm_skinny_residual_tiled"] == 0
        assert calls["sia_rope_kv_write"] == layers and calls["sia_add_rmsnorm"] == 2 * layers + 1
        for name in counted:
            calls[name] = 0
        runner.run([StepEntry("r", tokens[37:], [2])])        # three tokens
        assert calls["sia_gemm_skinny_rope"] == layers and calls["sia_gemm_skinny_swiglu"] == layers
        # (from the weight as it is or from the kernels' own copy of it; the last product waits for the rows that are wanted)
        assert calls["sia_gemm_skinny_residual"] + calls["sia_gemm_skinny_residual_tiled"] == 2 * layers - 1
        assert calls["sia_rope_kv_write"] == 0 and calls["sia_add_rmsnorm"] == 2   # the first norm and the last
    finally:
        for name in counted:
            setattr(core, name, real[name])
        cache.release("r")
