"""Parts that are not the served architecture's, defined here and plugged in from outside.

A toy mixer with state of its own, a layer order that names a layer twice, and a mixer that reads
another layer's pages are registered, built and stepped without a change to the package's files;
so are a feed-forward that routes tokens to experts, a norm and a position encoding of other kinds.
They run on the CPU with the torch twins and on the GPU with the HIP kernels.
"""


import pytest
import torch

from helpers import rel_err
from simple_inference_amd.cache import CacheManager
from simple_inference_amd.config import EngineConfig, register_architecture, unregister_architecture
from simple_inference_amd.engine import StepEntry, StepRunner, build_model
from simple_inference_amd.parts import (
    MIXERS, LayerSpec, ModelPlan, PartSpec, StateNeed, TensorSpec, register_mixer,
)
from simple_inference_amd.weights import random_tensors, target_dtype

BACKENDS = [pytest.param("twins"), pytest.param("hip-f32", marks=pytest.mark.gpu),
            pytest.param("hip-bf16", marks=pytest.mark.gpu)]


class RunningMeanMixer:
    """out[t] = W . mean(h[0..t]): the state is the running sum of the inputs, one row per request."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.env = env
        self.w = None

    def weight_specs(self):
        return {"w": TensorSpec((self.hidden, self.hidden))}

    def bind(self, tensors):
        self.w = tensors["w"]

    def cache_need(self):
        return None

    def state_need(self):
        return StateNeed((self.hidden,), "float32")

    def forward(self, h, ctx, cache):
        means = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        slots = ctx.state_slots.tolist()
        positions = ctx.positions.tolist()
        t = 0
        for s, n in enumerate(ctx.q_lens):
            running = cache.state[slots[s]]
            for i in range(n):
                running += h[t].float()
                means[t] = running / (positions[t] + 1)
                t += 1
        return self.env.kernels.linear(means.to(h.dtype), self.w)


H, V = 32, 64


def toy_plan(cfg):
    norm = lambda name: PartSpec("rmsnorm", {"size": H, "eps": 1e-5}, {"weight": name})
    ffn = lambda p: PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 48},
                             {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})
    rope = {"kind": "rope", "params": {"rotary_dim": 8, "theta": 10000.0, "scaling": None}}   # partial rotation
    attn = lambda p, **extra: PartSpec(
        "attention", dict({"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "position": rope}, **extra),
        {k: f"{p}.{k}" for k in (("q", "o") if "kv_from_layer" in extra else ("q", "k", "v", "o"))})
    layers = [
        LayerSpec(mixer=attn("l0.attn", window=cfg.get("window")), feed_forward=ffn("l0.ffn"),
                  mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2")),
        LayerSpec(mixer=PartSpec("test_running_mean", {"hidden_size": H}, {"w": "l1.mix.w"}), feed_forward=ffn("l1.ffn"),
                  mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2")),
        LayerSpec(mixer=attn("l2.attn", kv_from_layer=0, window=cfg.get("window")), feed_forward=ffn("l2.ffn"),
                  mixer_norm=norm("l2.n1"), feed_forward_norm=norm("l2.n2")),
    ]
    return ModelPlan(
        hidden_size=H, vocab_size=V,
        embedding=PartSpec("embedding", {"vocab_size": V, "hidden_size": H}, {"weight": "embed"}),
        layers=layers, order=cfg.get("order", [0, 1, 2, 1]),   # layer 1 runs twice; each run has a state of its own
        final_norm=norm("final"), head=PartSpec("head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}),
    )


@pytest.fixture()
def toy_registered():
    register_mixer("test_running_mean", RunningMeanMixer, replace=True)
    register_architecture("ToyForTests", lambda d: d, toy_plan, replace=True)
    yield
    unregister_architecture("ToyForTests")
    MIXERS.unregister("test_running_mean")


def make(backend, cfg, page_size=4, num_pages=32):
    if backend == "twins":
        from twins import TwinKernels
        kernels, device, dtype = TwinKernels(), "cpu", "float32"
    else:
        from simple_inference_amd.kernels import HipKernels
        kernels, device = HipKernels(), "cuda:0"
        dtype = "float32" if backend == "hip-f32" else "bfloat16"
    ecfg = EngineConfig(device=device, dtype=dtype, max_seq_len=128, block_size=page_size, max_running=3)
    model, _ = build_model(cfg, ecfg, kernels)
    expected = model.expected_tensors()
    drawn = random_tensors(expected, seed=3, std=0.15, gain_std=0.1)
    model.bind({k: t.to(device=device, dtype=target_dtype(t.dtype, expected[k].role, ecfg.torch_dtype))
                for k, t in drawn.items()})
    cache = CacheManager(model.cache_layout(), page_size=page_size, num_pages=num_pages, max_running=3,
                         dtype=ecfg.torch_dtype, device=device)
    return StepRunner(model, cache, kernels, device, 128), cache, drawn


def toy_reference(w, tokens, order, window):
    """The toy model, whole sequence, in float64, written out plainly."""
    import plain_llama as plain
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    x = w["embed"][tokens]
    pos = torch.arange(T)
    inv = plain.rope_inv_freq(8, 10000.0)
    cos, sin = plain.rope_tables(pos, inv, torch.float64)

    def rot(t):  # the first 8 of 16 dims rotate
        return torch.cat([plain.apply_rope(t[..., :8], cos, sin), t[..., 8:]], dim=-1)

    kv0 = None
    for li in order:
        p = f"l{li}"
        h = plain.rms_norm(x, w[f"{p}.n1"], 1e-5)
        if li == 1:
            mean = h.cumsum(0) / (pos[:, None] + 1)
            a = mean @ w["l1.mix.w"].T
        else:
            q = rot((h @ w[f"{p}.attn.q"].T).view(T, 4, 16))
            if li == 0:
                kv0 = (rot((h @ w["l0.attn.k"].T).view(T, 2, 16)), (h @ w["l0.attn.v"].T).view(T, 2, 16))
            a = plain.attention(q, kv0[0], kv0[1], pos, pos, window=window).reshape(T, 64) @ w[f"{p}.attn.o"].T
        x = x + a
        h = plain.rms_norm(x, w[f"{p}.n2"], 1e-5)
        x = x + plain.swiglu_mlp(h, w[f"{p}.ffn.gate"], w[f"{p}.ffn.up"], w[f"{p}.ffn.down"])
    return plain.rms_norm(x, w["final"], 1e-5) @ w["embed"].T


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("window", [None, 6])
def test_toy_architecture_is_registered_built_and_stepped(toy_registered, backend, window):
    cfg = {"architectures": ["ToyForTests"], "window": window}
    runner, cache, weights = make(backend, cfg)
    layout = runner.model.cache_layout()
    assert len(layout.states) == 2 and layout.run_state == [None, 0, None, 1]      # a state per run of layer 1
    assert layout.run_kv[0] == layout.run_kv[2] and layout.run_kv[1] is None          # layer 2 reads layer 0's pages
    assert layout.kv_slabs == [1]

    g = torch.Generator().manual_seed(0)
    seqs = {r: torch.randint(0, V, (n,), generator=g).tolist() for r, n in ((1, 23), (2, 9), (3, 15))}
    want = {r: toy_reference(weights, t, [0, 1, 2, 1], window) for r, t in seqs.items()}
    tol = 3e-2 if backend == "hip-bf16" else 2e-5

    # whole, alone
    for r, toks in seqs.items():
        cache.admit(r)
        out = runner.run([StepEntry(r, toks, list(range(len(toks))))])
        assert rel_err(out, want[r]) <= tol
        cache.release(r)
    # in portions, mixed with each other, slots and pages handed out again
    cuts = {1: [5, 1, 9, 2, 6], 2: [2, 7], 3: [1, 1, 13]}
    fed = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    for r in seqs:
        cache.admit(r)
    while any(cuts.values()):
        entries = []
        for r in seqs:
            if cuts[r]:
                n = cuts[r].pop(0)
                entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))))
                fed[r] += n
        out = runner.run(entries)
        i = 0
        for e in entries:
            got[e.req].append(out[i:i + len(e.tokens)])
            i += len(e.tokens)
    for r in seqs:
        assert rel_err(torch.cat(got[r]), want[r]) <= tol
        cache.release(r)
    cache.check()
    assert cache.free_pages() == 32 and cache.slots.free_slots == 3


@pytest.mark.parametrize("backend", BACKENDS)
def test_each_run_of_a_layer_has_pages_of_its_own(toy_registered, backend):
    """Order [0, 0, 1]: the attention layer runs twice; its second run must not see the keys of the first."""
    def plan(cfg):
        p = toy_plan(cfg)
        p.layers = p.layers[:2]
        p.order = [0, 0, 1]
        return p
    register_architecture("ToyTwice", lambda d: d, plan, replace=True)
    try:
        runner, cache, weights = make(backend, {"architectures": ["ToyTwice"]})
        assert runner.model.cache_layout().kv_slabs == [2]
        toks = torch.randint(0, V, (19,), generator=torch.Generator().manual_seed(1)).tolist()

        import plain_llama as plain
        w = {k: v.double() for k, v in weights.items()}
        T, pos = len(toks), torch.arange(len(toks))
        inv = plain.rope_inv_freq(8, 10000.0)
        cos, sin = plain.rope_tables(pos, inv, torch.float64)
        rot = lambda t: torch.cat([plain.apply_rope(t[..., :8], cos, sin), t[..., 8:]], dim=-1)
        x = w["embed"][toks]
        for li in (0, 0):
            h = plain.rms_norm(x, w["l0.n1"], 1e-5)
            q, k = rot((h @ w["l0.attn.q"].T).view(T, 4, 16)), rot((h @ w["l0.attn.k"].T).view(T, 2, 16))
            v = (h @ w["l0.attn.v"].T).view(T, 2, 16)
            x = x + plain.attention(q, k, v, pos, pos).reshape(T, 64) @ w["l0.attn.o"].T
            x = x + plain.swiglu_mlp(plain.rms_norm(x, w["l0.n2"], 1e-5), w["l0.ffn.gate"], w["l0.ffn.up"], w["l0.ffn.down"])
        h = plain.rms_norm(x, w["l1.n1"], 1e-5)
        x = x + (h.cumsum(0) / (pos[:, None] + 1)) @ w["l1.mix.w"].T
        x = x + plain.swiglu_mlp(plain.rms_norm(x, w["l1.n2"], 1e-5), w["l1.ffn.gate"], w["l1.ffn.up"], w["l1.ffn.down"])
        want = plain.rms_norm(x, w["final"], 1e-5) @ w["embed"].T

        cache.admit(1)
        got = torch.cat([runner.run([StepEntry(1, toks[a:b], list(range(b - a)))])
                         for a, b in ((0, 7), (7, 8), (8, 19))])
        assert rel_err(got, want) <= (3e-2 if backend == "hip-bf16" else 2e-5)
    finally:
        unregister_architecture("ToyTwice")


# ---- a feed-forward with routing, a norm and a position encoding of other kinds, from outside --------------------
class TopOneExperts:
    """Two small expert matrices and a router: every token goes through the expert its router score prefers,
    weighted by the softmax of the two scores (float32 routing)."""

    def __init__(self, params, env):
        self.hidden, self.n = int(params["hidden_size"]), int(params["experts"])
        self.env = env

    def weight_specs(self):
        specs = {"router": TensorSpec((self.n, self.hidden))}
        for e in range(self.n):
            specs[f"expert{e}"] = TensorSpec((self.hidden, self.hidden))
        return specs

    def bind(self, tensors):
        self.router = tensors["router"]
        self.experts = [tensors[f"expert{e}"] for e in range(self.n)]

    def forward(self, h, ctx):
        k = self.env.kernels
        scores = k.linear(h, self.router, out_float32=True)
        probs = torch.softmax(scores.float(), dim=-1)
        choice = probs.argmax(dim=-1)
        out = torch.zeros_like(h)
        for e, w in enumerate(self.experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                y = k.linear(h[rows].contiguous(), w)
                out[rows] = (y.float() * probs[rows, e:e + 1]).to(h.dtype)
        return out


class CenteredNorm:
    """A norm that also takes the mean away (the package's takes none): same contract towards the stream."""

    def __init__(self, params, env):
        self.size, self.eps, self.env = int(params["size"]), float(params["eps"]), env

    def weight_specs(self):
        return {"weight": TensorSpec((self.size,), "vector")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, stream, rows=None):
        if rows is None:
            if stream.delta is not None:
                stream.residual.add_(stream.delta.float())
                stream.delta = None
            x = stream.residual
        else:
            x = stream.residual[rows.long()]
            if stream.delta is not None:
                x = x + stream.delta[rows.long()].float()
        x = x - x.mean(-1, keepdim=True)
        return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight).to(self.env.dtype)


class LinearAngles:
    """Rotation angles that grow with the pair's index: angle(p, i) = p * step * (i + 1)."""

    def __init__(self, params, env):
        self.rotary_dim, self.step = int(params["rotary_dim"]), float(params["step"])
        self.env = env

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def tables(self):
        pos = torch.arange(self.env.max_positions, dtype=torch.float32)
        ang = torch.outer(pos, self.step * torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float32))
        return ang.cos().to(self.env.device).contiguous(), ang.sin().to(self.env.device).contiguous()


def other_kinds_plan(cfg):
    from simple_inference_amd.parts import PartSpec as P
    norm = lambda name: P("test_centered", {"size": H, "eps": 1e-4}, {"weight": name})
    pos = {"kind": "test_linear_angles", "params": {"rotary_dim": 16, "step": 0.05}}
    layer = LayerSpec(
        mixer=P("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "position": pos},
                {k: f"attn.{k}" for k in ("q", "k", "v", "o")}),
        feed_forward=P("test_top_one", {"hidden_size": H, "experts": 2},
                       {"router": "ffn.router", "expert0": "ffn.e0", "expert1": "ffn.e1"}),
        mixer_norm=norm("n1"), feed_forward_norm=norm("n2"))
    return ModelPlan(hidden_size=H, vocab_size=V,
                     embedding=P("embedding", {"vocab_size": V, "hidden_size": H}, {"weight": "embed"}),
                     layers=[layer], order=[0, 0], final_norm=norm("final"),
                     head=P("head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))


def other_kinds_reference(w, tokens):
    import plain_llama as plain
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    pos = torch.arange(T)
    ang = torch.outer(pos.double(), 0.05 * torch.arange(1, 9).double())
    cos, sin = torch.cat([ang.cos()] * 2, -1), torch.cat([ang.sin()] * 2, -1)

    def norm(x, g):
        x = x - x.mean(-1, keepdim=True)
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-4) * g

    x = w["embed"][tokens]
    for _ in range(2):
        h = norm(x, w["n1"])
        q = plain.apply_rope((h @ w["attn.q"].T).view(T, 2, 16), cos, sin)
        k = plain.apply_rope((h @ w["attn.k"].T).view(T, 1, 16), cos, sin)
        v = (h @ w["attn.v"].T).view(T, 1, 16)
        x = x + plain.attention(q, k, v, pos, pos).reshape(T, 32) @ w["attn.o"].T
        h = norm(x, w["n2"])
        probs = torch.softmax(h @ w["ffn.router"].T, -1)
        choice = probs.argmax(-1)
        y = torch.stack([(h[t] @ w[f"ffn.e{int(choice[t])}"].T) * probs[t, choice[t]] for t in range(T)])
        x = x + y
    return norm(x, w["final"]) @ w["embed"].T


@pytest.mark.parametrize("backend", [pytest.param("twins"), pytest.param("hip-f32", marks=pytest.mark.gpu)])
def test_feed_forward_norm_and_position_encoding_of_other_kinds(backend):
    from simple_inference_amd.parts import (
        FEED_FORWARDS, NORMS, POSITION_ENCODINGS, register_feed_forward, register_norm, register_position_encoding,
    )
    register_feed_forward("test_top_one", TopOneExperts, replace=True)
    register_norm("test_centered", CenteredNorm, replace=True)
    register_position_encoding("test_linear_angles", LinearAngles, replace=True)
    register_architecture("ToyOtherKinds", lambda d: d, other_kinds_plan, replace=True)
    try:
        runner, cache, weights = make(backend, {"architectures": ["ToyOtherKinds"]})
        tokens = torch.randint(0, V, (23,), generator=torch.Generator().manual_seed(5)).tolist()
        ref = other_kinds_reference(weights, tokens)
        cache.admit(1)
        got, fed = [], 0
        for n in (9, 2, 1, 1, 7, 3):           # portions and single tokens, as for any architecture
            got.append(runner.run([StepEntry(1, tokens[fed:fed + n], list(range(n)))]))
            fed += n
        assert rel_err(torch.cat(got), ref) < 3e-5
        cache.release(1)
        cache.check()
    finally:
        unregister_architecture("ToyOtherKinds")
        FEED_FORWARDS.unregister("test_top_one")
        NORMS.unregister("test_centered")
        POSITION_ENCODINGS.unregister("test_linear_angles")


# ---- an embedding and a head of other kinds, a cache of two widths, a state that does not start at zero ----------
class ScaledEmbedding:
    """Rows of the table times a constant (as some architectures scale their embeddings by sqrt(hidden))."""

    def __init__(self, params, env):
        self.vocab, self.hidden, self.factor = int(params["vocab_size"]), int(params["hidden_size"]), float(params["factor"])
        self.env = env

    def weight_specs(self):
        return {"weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, ctx):
        return self.env.kernels.embed(ctx.token_ids, self.weight) * self.factor


class SoftCappedHead:
    """logits = cap * tanh(h W^T / cap), with a matrix of its own or the embedding's."""

    def __init__(self, params, env):
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        self.cap, self.tied, self.env = float(params["cap"]), bool(params.get("tied")), env
        self.embedding = None

    def share_embedding(self, embedding):
        self.embedding = embedding

    def weight_specs(self):
        return {} if self.tied else {"weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.own = tensors.get("weight")

    def forward(self, h):
        w = self.embedding.weight if self.tied else self.own
        return self.cap * torch.tanh(self.env.kernels.linear(h, w, out_float32=True) / self.cap)


class RunningMaxMixer:
    """out[t] = W . max(h[0..t]) elementwise: a state that must start far below zero, not at it."""

    START = -1.0e30

    def __init__(self, params, env):
        self.hidden, self.env = int(params["hidden_size"]), env

    def weight_specs(self):
        return {"w": TensorSpec((self.hidden, self.hidden))}

    def bind(self, tensors):
        self.w = tensors["w"]

    def cache_need(self):
        return None

    def state_need(self):
        return StateNeed((self.hidden,), "float32", init=self.START)

    def forward(self, h, ctx, cache):
        out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        slots = ctx.state_slots.tolist()
        t = 0
        for s, n in enumerate(ctx.q_lens):
            running = cache.state[slots[s]]
            for _ in range(n):
                torch.maximum(running, h[t].float(), out=running)
                out[t] = running
                t += 1
        return self.env.kernels.linear(out.to(h.dtype), self.w)


class NarrowValueMixer:
    """Single-head attention without rotation whose cached values are narrower than its keys (as a mixer that
    caches a compressed value would have them): keys of 16, values of 8, written to and read from the pages here,
    with plain tensor operations.  The cache manager only has to give it pages of the two widths."""

    KEY, VALUE = 16, 8

    def __init__(self, params, env):
        self.hidden, self.env = int(params["hidden_size"]), env

    def weight_specs(self):
        return {"q": TensorSpec((self.KEY, self.hidden)), "k": TensorSpec((self.KEY, self.hidden)),
                "v": TensorSpec((self.VALUE, self.hidden)), "o": TensorSpec((self.hidden, self.VALUE))}

    def bind(self, tensors):
        self.w = tensors

    def cache_need(self):
        from simple_inference_amd.parts import PagedKVNeed
        return PagedKVNeed(1, self.KEY, None, value_head_dim=self.VALUE)

    def state_need(self):
        return None

    def forward(self, h, ctx, cache):
        lin = self.env.kernels.linear
        q, k, v = lin(h, self.w["q"]), lin(h, self.w["k"]), lin(h, self.w["v"])
        assert cache.k_pages.shape[1:] == (1, cache.page_size, self.KEY)
        assert cache.v_pages.shape[1:] == (1, self.VALUE, cache.page_size)
        out = torch.empty((h.shape[0], self.VALUE), dtype=torch.float32, device=h.device)
        positions, seqs = ctx.positions.tolist(), ctx.seq_of_token.tolist()
        for t, (p, s) in enumerate(zip(positions, seqs)):      # write first: a token sees itself
            page = int(cache.block_table[s, p // cache.page_size])
            cache.k_pages[page, 0, p % cache.page_size] = k[t]
            cache.v_pages[page, 0, :, p % cache.page_size] = v[t]
        for t, (p, s) in enumerate(zip(positions, seqs)):
            pages = cache.block_table[s, :p // cache.page_size + 1].long()
            keys = cache.k_pages[pages, 0].reshape(-1, self.KEY)[:p + 1].float()
            vals = cache.v_pages[pages, 0].permute(0, 2, 1).reshape(-1, self.VALUE)[:p + 1].float()
            probs = torch.softmax(keys @ q[t].float() / 4.0, dim=0)
            out[t] = probs @ vals
        return lin(out.to(h.dtype), self.w["o"])


def odd_ends_plan(cfg):
    from simple_inference_amd.parts import PartSpec as P
    norm = lambda name: P("rmsnorm", {"size": H, "eps": 1e-5}, {"weight": name})
    ffn = lambda p: P("swiglu", {"hidden_size": H, "intermediate_size": 48},
                      {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})
    layers = [
        LayerSpec(mixer=P("test_running_max", {"hidden_size": H}, {"w": "l0.w"}), feed_forward=ffn("l0.ffn"),
                  mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2")),
        LayerSpec(mixer=P("test_narrow_value", {"hidden_size": H}, {k: f"l1.{k}" for k in "qkvo"}),
                  feed_forward=ffn("l1.ffn"), mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2")),
    ]
    tied = bool(cfg.get("tied"))
    return ModelPlan(
        hidden_size=H, vocab_size=V,
        embedding=P("test_scaled_embedding", {"vocab_size": V, "hidden_size": H, "factor": 3.0}, {"weight": "embed"}),
        layers=layers, final_norm=norm("final"),
        head=P("test_soft_cap", {"vocab_size": V, "hidden_size": H, "cap": 2.0, "tied": tied},
               {} if tied else {"weight": "head"}))


def odd_ends_reference(w, tokens, tied):
    import plain_llama as plain
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    x = w["embed"][tokens] * 3.0
    h = plain.rms_norm(x, w["l0.n1"], 1e-5)
    x = x + torch.cummax(h, dim=0).values @ w["l0.w"].T
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["l0.n2"], 1e-5), w["l0.ffn.gate"], w["l0.ffn.up"], w["l0.ffn.down"])
    h = plain.rms_norm(x, w["l1.n1"], 1e-5)
    q, k, v = h @ w["l1.q"].T, h @ w["l1.k"].T, h @ w["l1.v"].T
    scores = (q @ k.T / 4.0).masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    x = x + (torch.softmax(scores, -1) @ v) @ w["l1.o"].T
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["l1.n2"], 1e-5), w["l1.ffn.gate"], w["l1.ffn.up"], w["l1.ffn.down"])
    logits = plain.rms_norm(x, w["final"], 1e-5) @ (w["embed"] if tied else w["head"]).T
    return 2.0 * torch.tanh(logits / 2.0)


@pytest.fixture()
def odd_ends_registered():
    from simple_inference_amd.parts import EMBEDDINGS, HEADS, register_embedding, register_head
    register_embedding("test_scaled_embedding", ScaledEmbedding, replace=True)
    register_head("test_soft_cap", SoftCappedHead, replace=True)
    register_mixer("test_running_max", RunningMaxMixer, replace=True)
    register_mixer("test_narrow_value", NarrowValueMixer, replace=True)
    register_architecture("ToyOddEnds", lambda d: d, odd_ends_plan, replace=True)
    yield
    unregister_architecture("ToyOddEnds")
    EMBEDDINGS.unregister("test_scaled_embedding")
    HEADS.unregister("test_soft_cap")
    MIXERS.unregister("test_running_max")
    MIXERS.unregister("test_narrow_value")


@pytest.mark.parametrize("backend", [pytest.param("twins"), pytest.param("hip-f32", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("tied", [False, True])
def test_embedding_head_cache_widths_and_initial_state_from_outside(odd_ends_registered, backend, tied):
    """An embedding that scales, a head that caps its logits (with a matrix of its own, or tied), a mixer whose
    cached values are narrower than its keys and a state that starts at -1e30: all registered here, none known to
    the package, stepped in portions beside each other with slots and pages handed out again."""
    runner, cache, weights = make(backend, {"architectures": ["ToyOddEnds"], "tied": tied})
    group = cache.groups[0]
    assert group.need.head_dim == 16 and group.need.value_dim == 8
    assert group.k.shape[-1] == 16 and group.v.shape[-2] == 8
    g = torch.Generator().manual_seed(2)
    seqs = {r: torch.randint(0, V, (n,), generator=g).tolist() for r, n in ((1, 14), (2, 21), (3, 6), (4, 11))}
    want = {r: odd_ends_reference(weights, t, tied) for r, t in seqs.items()}
    cuts = {1: [5, 1, 8], 2: [2, 7, 1, 11], 3: [6], 4: [1, 10]}
    got, fed, live, waiting = {r: [] for r in seqs}, {r: 0 for r in seqs}, [], list(seqs)
    while waiting or live:
        while waiting and len(live) < 3:        # three slots for four requests: one is used a second time
            live.append(waiting.pop(0))
            cache.admit(live[-1])
        entries = []
        for r in live:
            n = cuts[r].pop(0)
            entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
        out = runner.run(entries)
        i = 0
        for e in entries:
            got[e.req].append(out[i:i + len(e.tokens)])
            i += len(e.tokens)
        for r in [r for r in live if not cuts[r]]:
            cache.release(r)
            live.remove(r)
    for r in seqs:
        assert rel_err(torch.cat(got[r]), want[r]) <= 3e-5, r
    cache.check()
    assert cache.free_pages() == 32 and cache.slots.free_slots == 3


def test_trace_replay_runs_an_architecture_whose_configuration_is_a_plain_dictionary(toy_registered, tmp_path):
    """The replay program's driver takes the architecture from config.json alone: a registered toy whose
    parse_config returns the dictionary itself is replayed like any other model."""
    from simple_inference_amd.replay import TraceReplayer
    from simple_inference_amd.weights import write_model_folder
    from twins import TwinKernels
    cfg = {"architectures": ["ToyForTests"], "window": None, "max_position_embeddings": 256}
    model, _ = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    weights = random_tensors(model.expected_tensors(), seed=3, std=0.15, gain_std=0.1)
    folder = write_model_folder(tmp_path, cfg, weights)
    rp = TraceReplayer(folder, "float32", 64, block_size=16, device="cpu", kernels=TwinKernels())
    assert rp.describe().startswith("ToyForTests")
    tokens = torch.randint(0, V, (23,), generator=torch.Generator().manual_seed(0)).tolist()
    want = toy_reference(weights, tokens, [0, 1, 2, 1], None)
    got = [rp.step([{"id": "a", "tokens": tokens[a:b], "want": list(range(b - a))}], ["a"] if b == 23 else [])
           for a, b in ((0, 9), (9, 11), (11, 12), (12, 23))]
    assert rel_err(torch.cat(got), want) <= 2e-5
    assert not rp.ids and rp.cache.free_pages() == 4


def test_a_head_size_no_kernel_takes_is_refused_when_the_model_is_built():
    """Not at the first launch: the mixer asks the kernels when it is built."""
    class Kernels:
        def check_attention_geometry(self, n_heads, n_kv_heads, head_dim):
            if head_dim > 256:
                raise ValueError(f"head size {head_dim} is outside what the attention kernels take")
    from helpers import TINY_A
    cfg = dict(TINY_A, head_dim=320)
    with pytest.raises(ValueError, match="head size 320"):
        build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=Kernels())
    build_model(dict(TINY_A, head_dim=256), EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=Kernels())


@pytest.mark.gpu
def test_the_compiled_kernels_refuse_a_head_size_beyond_their_limit_at_build_time():
    from helpers import TINY_A
    from simple_inference_amd.kernels import HipKernels, KernelError
    with pytest.raises(KernelError, match="head size 272"):
        build_model(dict(TINY_A, head_dim=272), EngineConfig(device="cuda:0", dtype="bfloat16", max_seq_len=64), HipKernels())


# ---- a position encoding with a second axis, brought by the step's entries ------------------------------------------
class TwoAxisAngles:
    """Half of the rotary pairs turn with the token's position, the other half with a second number per token that the
    caller brings (``StepEntry.extra["column"]``), as encodings for grids of patches do.  The package's rotation
    kernel takes one table row per token, so this encoding hands its mixer a table indexed by a *combined* index
    and says how to form it; here the toy mixer below forms it."""

    def __init__(self, params, env):
        self.rotary_dim, self.columns, self.env = int(params["rotary_dim"]), int(params["columns"]), env

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def angles(self, positions, columns):
        quarter = self.rotary_dim // 4
        freq = 1.0 / (100.0 ** (torch.arange(quarter, dtype=torch.float32) / quarter))
        return torch.cat([positions.float()[:, None] * freq, columns.float()[:, None] * freq], dim=-1)   # [N, rotary/2]


class TwoAxisMixer:
    """out = W_o . rotate(W_q h) with the two-axis angles: no attention, so that the test is about the step's
    metadata reaching a part, nothing else."""

    def __init__(self, params, env):
        self.hidden, self.env = int(params["hidden_size"]), env
        self.position = TwoAxisAngles({"rotary_dim": self.hidden, "columns": 8}, env)

    def weight_specs(self):
        return {"q": TensorSpec((self.hidden, self.hidden)), "o": TensorSpec((self.hidden, self.hidden))}

    def bind(self, tensors):
        self.w = tensors

    def cache_need(self):
        return None

    def state_need(self):
        return None

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        q = k.linear(h, self.w["q"]).float()
        ang = self.position.angles(ctx.positions.cpu(), ctx.extra["column"].cpu()).to(q.device)
        half = self.hidden // 2
        a, b = q[:, :half], q[:, half:]
        rotated = torch.cat([a * ang.cos() - b * ang.sin(), b * ang.cos() + a * ang.sin()], dim=-1)
        return k.linear(rotated.to(h.dtype), self.w["o"])


def test_a_second_position_axis_reaches_a_part_through_the_step(tmp_path):
    """Entries bring a number per token beside the token id; the step function lays it out with the batch
    (sequences that bring one token first) and hands it to the parts as ``ctx.extra``."""
    def plan(cfg):
        from simple_inference_amd.parts import PartSpec as P
        norm = lambda name: P("rmsnorm", {"size": H, "eps": 1e-5}, {"weight": name})
        layer = LayerSpec(mixer=P("test_two_axis", {"hidden_size": H}, {"q": "q", "o": "o"}),
                          feed_forward=P("swiglu", {"hidden_size": H, "intermediate_size": 48},
                                         {"gate": "gate", "up": "up", "down": "down"}),
                          mixer_norm=norm("n1"), feed_forward_norm=norm("n2"))
        return ModelPlan(hidden_size=H, vocab_size=V,
                         embedding=P("embedding", {"vocab_size": V, "hidden_size": H}, {"weight": "embed"}),
                         layers=[layer], final_norm=norm("final"),
                         head=P("head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))
    register_mixer("test_two_axis", TwoAxisMixer, replace=True)
    register_architecture("ToyTwoAxis", lambda d: d, plan, replace=True)
    try:
        import plain_llama as plain
        runner, cache, weights = make("twins", {"architectures": ["ToyTwoAxis"]})
        w = {k: v.double() for k, v in weights.items()}
        g = torch.Generator().manual_seed(4)
        seqs = {r: (torch.randint(0, V, (n,), generator=g).tolist(), torch.randint(0, 8, (n,), generator=g).tolist())
                for r, n in ((1, 9), (2, 1), (3, 6))}

        def reference(tokens, columns):
            T = len(tokens)
            x = w["embed"][tokens]
            q = plain.rms_norm(x, w["n1"], 1e-5) @ w["q"].T
            quarter = H // 4
            freq = (1.0 / (100.0 ** (torch.arange(quarter, dtype=torch.float32) / quarter))).double()
            ang = torch.cat([torch.arange(T).double()[:, None] * freq, torch.tensor(columns).double()[:, None] * freq], -1)
            a, b = q[:, :H // 2], q[:, H // 2:]
            x = x + torch.cat([a * ang.cos() - b * ang.sin(), b * ang.cos() + a * ang.sin()], -1) @ w["o"].T
            x = x + plain.swiglu_mlp(plain.rms_norm(x, w["n2"], 1e-5), w["gate"], w["up"], w["down"])
            return plain.rms_norm(x, w["final"], 1e-5) @ w["embed"].T

        for r in seqs:
            cache.admit(r)
        # first step: a portion of 1, the single token of 2, a portion of 3 (the step sorts 2 to the front)
        first = [StepEntry(1, seqs[1][0][:4], [0, 3], extra={"column": seqs[1][1][:4]}),
                 StepEntry(2, seqs[2][0], [0], extra={"column": seqs[2][1]}),
                 StepEntry(3, seqs[3][0][:5], [4], extra={"column": seqs[3][1][:5]})]
        out = runner.run(first)
        want = torch.stack([reference(*seqs[1])[0], reference(*seqs[1])[3], reference(*seqs[2])[0], reference(*seqs[3])[4]])
        assert rel_err(out, want) <= 2e-5
        second = [StepEntry(3, seqs[3][0][5:], [0], extra={"column": seqs[3][1][5:]}),
                  StepEntry(1, seqs[1][0][4:], [4], extra={"column": seqs[1][1][4:]})]
        out = runner.run(second)
        assert rel_err(out, torch.stack([reference(*seqs[3])[5], reference(*seqs[1])[8]])) <= 2e-5
        with pytest.raises(ValueError, match="column"):     # every entry of a step must bring it, or none
            runner.run([StepEntry(2, [1], [0]), StepEntry(3, [2], [0], extra={"column": [1]})])
        assert cache.lengths[2] == 1 and cache.lengths[3] == 6      # the refused step took nothing
    finally:
        unregister_architecture("ToyTwoAxis")
        MIXERS.unregister("test_two_axis")


# ---- blocks of other kinds: a third norm, no feed-forward, no mixer -------------------------------------------------
class SandwichBlock:
    """x += post_norm(mixer(norm1(x))); x += feed_forward(norm2(x)): a block with three norms, of which one
    normalises a part's output before it is added.  It takes its parts under names of its own choosing."""

    def __init__(self, mixer, feed_forward, mixer_norm, after_mixer_norm, feed_forward_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.after_mixer_norm, self.feed_forward_norm = mixer_norm, after_mixer_norm, feed_forward_norm

    def forward(self, stream, ctx, cache):
        from simple_inference_amd.parts.context import ResidualStream
        h = self.mixer_norm.forward(stream)
        mixed = self.mixer.forward(h, ctx, cache)
        mixed = mixed.compute() if hasattr(mixed, "compute") else mixed
        # the norm of the output: a stream of its own whose residual is the output itself
        stream.delta = self.after_mixer_norm.forward(ResidualStream(mixed.float()))
        h = self.feed_forward_norm.forward(stream)
        stream.delta = self.feed_forward.forward(h, ctx)


class MixerOnlyBlock:
    """x += mixer(norm(x)), and nothing else."""

    def __init__(self, mixer, norm):
        self.mixer, self.norm = mixer, norm

    def forward(self, stream, ctx, cache):
        stream.delta = self.mixer.forward(self.norm.forward(stream), ctx, cache)


class FeedForwardOnlyBlock:
    """x += feed_forward(norm(x)): a layer without a mixer owns no pages and no state."""

    def __init__(self, feed_forward, norm):
        self.feed_forward, self.norm = feed_forward, norm

    def forward(self, stream, ctx, cache):
        assert cache.k_pages is None and cache.state is None
        stream.delta = self.feed_forward.forward(self.norm.forward(stream), ctx)


def other_blocks_plan(cfg):
    P = PartSpec
    norm = lambda name: P("rmsnorm", {"size": H, "eps": 1e-5}, {"weight": name}, role="norm")
    rope = {"kind": "rope", "params": {"rotary_dim": 16, "theta": 10000.0, "scaling": None}}
    attn = lambda p: P("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 2, "head_dim": 16, "position": rope},
                       {k: f"{p}.{k}" for k in "qkvo"}, role="mixer")
    ffn = lambda p: P("swiglu", {"hidden_size": H, "intermediate_size": 48},
                      {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"}, role="feed_forward")
    layers = [
        LayerSpec(block="test_sandwich", mixer=attn("l0.attn"), feed_forward=ffn("l0.ffn"), mixer_norm=norm("l0.n1"),
                  feed_forward_norm=norm("l0.n2"), parts={"after_mixer_norm": norm("l0.n3")}),
        LayerSpec(block="test_mixer_only", parts={"mixer": attn("l1.attn"), "norm": norm("l1.n")}),
        LayerSpec(block="test_feed_forward_only", parts={"feed_forward": ffn("l2.ffn"), "norm": norm("l2.n")}),
    ]
    return ModelPlan(hidden_size=H, vocab_size=V,
                     embedding=P("embedding", {"vocab_size": V, "hidden_size": H}, {"weight": "embed"}),
                     layers=layers, order=[0, 2, 1, 2], final_norm=norm("final"),
                     head=P("head", {"vocab_size": V, "hidden_size": H, "tied": True}, {}))


def other_blocks_reference(w, tokens):
    import plain_llama as plain
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    pos = torch.arange(T)
    cos, sin = plain.rope_tables(pos, plain.rope_inv_freq(16, 10000.0), torch.float64)
    norm = lambda x, name: plain.rms_norm(x, w[name], 1e-5)

    def attend(h, p):
        q = plain.apply_rope((h @ w[f"{p}.q"].T).view(T, 2, 16), cos, sin)
        k = plain.apply_rope((h @ w[f"{p}.k"].T).view(T, 2, 16), cos, sin)
        v = (h @ w[f"{p}.v"].T).view(T, 2, 16)
        return plain.attention(q, k, v, pos, pos).reshape(T, 32) @ w[f"{p}.o"].T

    ffn = lambda h, p: plain.swiglu_mlp(h, w[f"{p}.gate"], w[f"{p}.up"], w[f"{p}.down"])
    x = w["embed"][tokens]
    x = x + norm(attend(norm(x, "l0.n1"), "l0.attn"), "l0.n3")
    x = x + ffn(norm(x, "l0.n2"), "l0.ffn")
    x = x + ffn(norm(x, "l2.n"), "l2.ffn")
    x = x + attend(norm(x, "l1.n"), "l1.attn")
    x = x + ffn(norm(x, "l2.n"), "l2.ffn")
    return norm(x, "final") @ w["embed"].T


@pytest.mark.parametrize("backend", BACKENDS)
def test_blocks_with_a_third_norm_without_a_feed_forward_and_without_a_mixer(backend):
    """A layer is a block kind and the named parts that kind arranges: three block kinds defined here take parts
    under names of their own (a third norm; a mixer and one norm; a feed-forward and one norm), are registered
    from outside and run beside one another in one model.  The layer without a mixer owns no pages."""
    from simple_inference_amd.parts import BLOCKS, register_block
    for kind, cls in (("test_sandwich", SandwichBlock), ("test_mixer_only", MixerOnlyBlock),
                      ("test_feed_forward_only", FeedForwardOnlyBlock)):
        register_block(kind, cls, replace=True)
    register_architecture("ToyOtherBlocks", lambda d: d, other_blocks_plan, replace=True)
    try:
        runner, cache, weights = make(backend, {"architectures": ["ToyOtherBlocks"]})
        layout = runner.model.cache_layout()
        assert layout.run_kv == [(0, 0), None, (0, 1), None] and layout.kv_slabs == [2] and not layout.states
        tokens = torch.randint(0, V, (21,), generator=torch.Generator().manual_seed(8)).tolist()
        ref = other_blocks_reference(weights, tokens)
        cache.admit(1)
        got, fed = [], 0
        for n in (8, 1, 2, 1, 6, 3):
            got.append(runner.run([StepEntry(1, tokens[fed:fed + n], list(range(n)))]))
            fed += n
        assert rel_err(torch.cat(got), ref) < (2.5e-2 if backend == "hip-bf16" else 3e-5)
        cache.release(1)
        cache.check()
        # a block kind is told by name which parts it does not take
        register_architecture("ToyWrongParts", lambda d: d, lambda cfg: ModelPlan(
            hidden_size=H, vocab_size=V, embedding=other_blocks_plan(cfg).embedding,
            layers=[LayerSpec(block="test_mixer_only", mixer=other_blocks_plan(cfg).layers[1].parts["mixer"])],
            final_norm=other_blocks_plan(cfg).final_norm, head=other_blocks_plan(cfg).head), replace=True)
        with pytest.raises(ValueError, match="test_mixer_only.*does not take the parts"):
            make(backend, {"architectures": ["ToyWrongParts"]})
    finally:
        unregister_architecture("ToyOtherBlocks")
        unregister_architecture("ToyWrongParts")
        for kind in ("test_sandwich", "test_mixer_only", "test_feed_forward_only"):
            BLOCKS.unregister(kind)


def test_a_layer_spec_says_what_is_wrong_with_its_parts():
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5}, {"weight": "n"})
    with pytest.raises(ValueError, match="role"):
        LayerSpec(block="x", parts={"some_norm": norm})                       # a free name needs a role
    mixer = PartSpec("attention", {}, {}, role="mixer")
    with pytest.raises(ValueError, match="at most one"):
        LayerSpec(block="x", mixer=mixer, parts={"second": PartSpec("attention", {}, {}, role="mixer")})
    with pytest.raises(ValueError, match="twice"):
        LayerSpec(block="x", mixer=mixer, parts={"mixer": mixer})
    spec = LayerSpec(mixer=mixer, parts={"mixer_norm": norm})                # the four known names carry their roles
    assert spec.parts["mixer_norm"].role == "norm" and spec.mixer_norm is spec.parts["mixer_norm"]
    assert list(spec.parts) == ["mixer_norm", "mixer"]
