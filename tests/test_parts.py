"""Each part alone against the plain implementation's function for it, at sizes of its own."""


import pytest
import torch

import plain_llama as plain
from helpers import rel_err
from simple_inference_amd.cache import CacheManager
from simple_inference_amd.engine.step import StepEntry, StepRunner
from simple_inference_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, BuildEnv, ResidualStream
from simple_inference_amd.parts.embedding import OutputHead, TokenEmbedding
from simple_inference_amd.parts.model import CacheLayout

BACKENDS = [pytest.param("twins"), pytest.param("hip-f32", marks=pytest.mark.gpu),
            pytest.param("hip-bf16", marks=pytest.mark.gpu)]


def env_for(backend, max_positions=256):
    if backend == "twins":
        from twins import TwinKernels
        return BuildEnv(TwinKernels(), torch.device("cpu"), torch.float32, max_positions)
    from simple_inference_amd.kernels import HipKernels
    dtype = torch.float32 if backend == "hip-f32" else torch.bfloat16
    return BuildEnv(HipKernels(), torch.device("cuda:0"), dtype, max_positions)


def tol(backend):
    return 2e-2 if backend == "hip-bf16" else 1e-5


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def on(env, t, matrix=True):
    """A tensor as the loader would hand it to a part: matrices in the compute dtype, vectors in float32."""
    return t.to(device=env.device, dtype=env.dtype if matrix else torch.float32).contiguous()


def as_ref(env, t):
    """The same numbers the part sees, in float64 for the plain function."""
    return t.to(env.dtype).double()


class OneSequence:
    """A step context and cache for one whole sequence of T tokens, made by the package's own runner pieces."""

    def __init__(self, env, T, need=None, page_size=8):
        layout = CacheLayout()
        if need is not None:
            layout.kv_groups, layout.kv_slabs, layout.run_kv = [need], [1], [(0, 0)]
        else:
            layout.run_kv = [None]
        layout.run_state = [None]
        self.cache = CacheManager(layout, page_size=page_size, num_pages=64, max_running=2, dtype=env.dtype,
                                  device=env.device)

        class _M:  # the runner only asks a model for its vocabulary here
            vocab_size = 1 << 30
        runner = StepRunner(_M(), self.cache, env.kernels, env.device, 256)
        self.cache.admit(1)
        self.ctx = runner.build_context([StepEntry(1, [0] * T, [])])
        self.layer_cache = self.cache.layer_caches(self.ctx.block_tables)[0]


@pytest.mark.parametrize("backend", BACKENDS)
def test_norm_part(backend):
    env = env_for(backend)
    part = NORMS.get("rmsnorm")({"size": 200, "eps": 2e-5}, env)
    assert {k: v.shape for k, v in part.weight_specs().items()} == {"weight": (200,)}
    w, res, delta = 1 + rnd(200, seed=1, scale=0.2), rnd(6, 200, seed=2, scale=2.0), rnd(6, 200, seed=3)
    part.bind({"weight": on(env, w, matrix=False)})
    stream = ResidualStream(res.clone().to(env.device), on(env, delta))
    out = part.forward(stream)
    want = plain.rms_norm(res.double() + as_ref(env, delta), w.double(), 2e-5)
    assert rel_err(out, want) <= tol(backend)
    assert stream.delta is None and rel_err(stream.residual, res.double() + as_ref(env, delta)) <= 1e-6


@pytest.mark.parametrize("backend", BACKENDS)
def test_position_encoding_part(backend):
    env = env_for(backend, max_positions=300)
    scaling = {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 2.0,
               "original_max_position_embeddings": 32}
    part = POSITION_ENCODINGS.get("rope")({"rotary_dim": 48, "theta": 25000.0, "scaling": scaling}, env)
    cos, sin = part.tables()
    assert cos.shape == (300, 24) and cos.dtype == torch.float32 and cos.device.type == env.device.type
    inv = plain.rope_inv_freq(48, 25000.0, scaling)
    pc, ps = plain.rope_tables(torch.arange(300), inv)
    assert torch.allclose(cos.cpu(), pc[:, :24], atol=1e-6) and torch.allclose(sin.cpu(), ps[:, :24], atol=1e-6)
    assert POSITION_ENCODINGS.get("none")({}, env).tables() == (None, None)


@pytest.mark.parametrize("backend", BACKENDS)
def test_feed_forward_part(backend):
    env = env_for(backend)
    part = FEED_FORWARDS.get("swiglu")({"hidden_size": 72, "intermediate_size": 200}, env)
    g, u, d, x = rnd(200, 72, seed=1, scale=0.2), rnd(200, 72, seed=2, scale=0.2), rnd(72, 200, seed=3, scale=0.2), rnd(9, 72, seed=4)
    part.bind({"gate": on(env, g), "up": on(env, u), "down": on(env, d)})
    out = part.forward(on(env, x), None)
    want = plain.swiglu_mlp(as_ref(env, x), as_ref(env, g), as_ref(env, u), as_ref(env, d))
    assert rel_err(out, want) <= tol(backend)


def attention_weights(env, H, Hq, Hkv, D, seed):
    w = {"q": rnd(Hq * D, H, seed=seed, scale=0.2), "k": rnd(Hkv * D, H, seed=seed + 1, scale=0.2),
         "v": rnd(Hkv * D, H, seed=seed + 2, scale=0.2), "o": rnd(H, Hq * D, seed=seed + 3, scale=0.2)}
    return w, {k: on(env, t) for k, t in w.items()}


@pytest.mark.parametrize("backend", BACKENDS)
def test_attention_part(backend):
    env = env_for(backend)
    H, Hq, Hkv, D, T = 80, 6, 2, 32, 45
    params = {"hidden_size": H, "num_heads": Hq, "num_kv_heads": Hkv, "head_dim": D,
              "position": {"kind": "rope", "params": {"rotary_dim": D, "theta": 10000.0, "scaling": None}}}
    part = MIXERS.get("attention")(params, env)
    w, w_dev = attention_weights(env, H, Hq, Hkv, D, seed=10)
    part.bind(w_dev)
    assert part.w_qkv.shape == ((Hq + 2 * Hkv) * D, H)            # the three projections are one matrix
    seq = OneSequence(env, T, part.cache_need())
    h = rnd(T, H, seed=20)
    out = part.forward(on(env, h), seq.ctx, seq.layer_cache)
    cfg = {"num_attention_heads": Hq, "num_key_value_heads": Hkv, "head_dim": D, "hidden_size": H}
    names = {f"p.self_attn.{k}_proj.weight": as_ref(env, t) for k, t in w.items()}
    want = plain.attention_layer(as_ref(env, h), torch.arange(T), names, "p", cfg, plain.rope_inv_freq(D, 10000.0))
    assert rel_err(out, want) <= tol(backend)


@pytest.mark.parametrize("backend", BACKENDS)
def test_block_part(backend):
    env = env_for(backend)
    H, Hq, Hkv, D, I, T = 64, 4, 4, 16, 96, 21
    attn = MIXERS.get("attention")({"hidden_size": H, "num_heads": Hq, "num_kv_heads": Hkv, "head_dim": D,
                                    "position": {"kind": "rope", "params": {"rotary_dim": D, "theta": 5e5, "scaling": None}}}, env)
    ffn = FEED_FORWARDS.get("swiglu")({"hidden_size": H, "intermediate_size": I}, env)
    n1, n2 = (NORMS.get("rmsnorm")({"size": H, "eps": 1e-6}, env) for _ in range(2))
    aw, aw_dev = attention_weights(env, H, Hq, Hkv, D, seed=30)
    fw = {"gate": rnd(I, H, seed=40, scale=0.2), "up": rnd(I, H, seed=41, scale=0.2), "down": rnd(H, I, seed=42, scale=0.2)}
    g1, g2 = 1 + rnd(H, seed=43, scale=0.1), 1 + rnd(H, seed=44, scale=0.1)
    attn.bind(aw_dev)
    ffn.bind({k: on(env, t) for k, t in fw.items()})
    n1.bind({"weight": on(env, g1, matrix=False)})
    n2.bind({"weight": on(env, g2, matrix=False)})
    block = BLOCKS.get("prenorm")(attn, ffn, n1, n2)
    seq = OneSequence(env, T, attn.cache_need())
    x = rnd(T, H, seed=50)
    stream = ResidualStream(x.clone().to(env.device).float().contiguous())
    block.forward(stream, seq.ctx, seq.layer_cache)
    got = stream.residual.double().cpu() + stream.delta.double().cpu()   # the last add is still pending
    w = {"model.layers.0.input_layernorm.weight": g1.double(), "model.layers.0.post_attention_layernorm.weight": g2.double()}
    w.update({f"model.layers.0.self_attn.{k}_proj.weight": as_ref(env, t) for k, t in aw.items()})
    w.update({f"model.layers.0.mlp.{k}_proj.weight": as_ref(env, t) for k, t in fw.items()})
    cfg = {"num_attention_heads": Hq, "num_key_value_heads": Hkv, "head_dim": D, "hidden_size": H, "rms_norm_eps": 1e-6}
    want = plain.block(x.double(), torch.arange(T), w, 0, cfg, plain.rope_inv_freq(D, 5e5))
    assert rel_err(got, want) <= tol(backend)


@pytest.mark.parametrize("backend", BACKENDS)
def test_embedding_and_head_parts(backend):
    env = env_for(backend)
    table = rnd(331, 40, seed=1)
    emb = TokenEmbedding({"vocab_size": 331, "hidden_size": 40}, env)
    emb.bind({"weight": on(env, table)})

    class Ctx:
        token_ids = torch.tensor([330, 0, 17, 17], dtype=torch.int32, device=env.device)
    out = emb.forward(Ctx())
    assert out.dtype == torch.float32 and torch.equal(out.cpu(), as_ref(env, table)[[330, 0, 17, 17]].float())
    tied = OutputHead({"vocab_size": 331, "hidden_size": 40, "tied": True}, env)
    with pytest.raises(ValueError):
        tied.bind({})                       # tied, and given no embedding to share
    tied.share_embedding(emb)
    tied.bind({})
    assert tied.weight_specs() == {} and tied.weight.data_ptr() == emb.weight.data_ptr()
    h = rnd(3, 40, seed=2)
    logits = tied.forward(on(env, h))
    assert logits.dtype == torch.float32 and rel_err(logits, as_ref(env, h) @ as_ref(env, table).T) <= tol(backend)
    own = rnd(331, 40, seed=3)
    untied = OutputHead({"vocab_size": 331, "hidden_size": 40, "tied": False}, env)
    untied.bind({"weight": on(env, own)})
    assert rel_err(untied.forward(on(env, h)), as_ref(env, h) @ as_ref(env, own).T) <= tol(backend)


def test_a_part_with_a_forward_of_its_own_no_longer_says_it_is_the_plain_one():
    """Kernels that run a whole block in one call trust what the block and its parts say they are (``plain_form``).
    A subclass that computes something else (a forward of its own) must not inherit that description, or steps of
    many rows would silently run the base class's arithmetic while steps of few rows run the subclass's."""
    from simple_inference_amd.parts.attention import Attention
    from simple_inference_amd.parts.block import PreNormBlock
    from simple_inference_amd.parts.norm import RMSNorm
    from simple_inference_amd.parts.swiglu import SwiGLU
    env = env_for("twins")
    rope = {"kind": "rope", "params": {"rotary_dim": 16, "theta": 10000.0, "scaling": None}}
    attn_params = {"hidden_size": 32, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "position": rope}

    class OtherAttention(Attention):
        def forward(self, h, ctx, cache):
            return 2 * super().forward(h, ctx, cache)

    class OtherNorm(RMSNorm):
        def forward(self, stream, rows=None, scaled_ok=False):
            return super().forward(stream, rows) + 1

    class OtherFeedForward(SwiGLU):
        def forward(self, h, ctx):
            return -super().forward(h, ctx)

    class OtherBlock(PreNormBlock):
        def forward(self, stream, ctx, cache):
            super().forward(stream, ctx, cache)

    def built(attn_cls, norm_cls, ff_cls, block_cls):
        mixer, ff = attn_cls(attn_params, env), ff_cls({"hidden_size": 32, "intermediate_size": 48}, env)
        n1, n2 = norm_cls({"size": 32, "eps": 1e-5}, env), norm_cls({"size": 32, "eps": 1e-5}, env)
        mixer.bind({k: rnd(*spec.shape, seed=1) for k, spec in mixer.weight_specs().items()})
        ff.bind({k: rnd(*spec.shape, seed=2) for k, spec in ff.weight_specs().items()})
        for n in (n1, n2):
            n.bind({"weight": torch.ones(32)})
        return block_cls(mixer=mixer, feed_forward=ff, mixer_norm=n1, feed_forward_norm=n2)

    whole = built(Attention, RMSNorm, SwiGLU, PreNormBlock).plain_form()
    assert whole["kind"] == "prenorm"
    assert [whole[k]["kind"] for k in ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")] == \
        ["rmsnorm", "paged_attention", "rmsnorm", "swiglu"]
    assert built(OtherAttention, RMSNorm, SwiGLU, PreNormBlock).plain_form()["mixer"] is None
    assert built(Attention, OtherNorm, SwiGLU, PreNormBlock).plain_form()["mixer_norm"] is None
    assert built(Attention, RMSNorm, OtherFeedForward, PreNormBlock).plain_form()["feed_forward"] is None
    assert built(Attention, RMSNorm, SwiGLU, OtherBlock).plain_form() is None
