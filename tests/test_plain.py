"""What fixes the plain implementation beside the reference's text.

Each test pins one formula of ``plain_llama`` by a library routine it must reduce to, by an
invariant, or by a vector that the reference's own tests hold, chosen so that a plausible
mistake (a wrong sign or pairing, eps outside the root, a norm in the wrong place, a mask off
by one) fails it.
"""

import math

import torch
import torch.nn.functional as F

import plain_llama as plain

torch.manual_seed(0)


# ---- rms norm -------------------------------------------------------------------------------
def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 48, dtype=torch.float64), torch.randn(48, dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)


def test_rms_norm_eps_inside_the_root_and_no_mean_subtraction():
    x = torch.full((1, 16), 1e-3, dtype=torch.float64)
    y = plain.rms_norm(x, torch.ones(16, dtype=torch.float64), 1e-2)
    assert torch.allclose(y, torch.full_like(y, 1e-3 / math.sqrt(1e-6 + 1e-2)))  # not 1e-3 / (1e-3 + eps)
    c = torch.full((1, 16), 3.0, dtype=torch.float64)  # a constant row keeps its value / rms = 1 (a layer norm gives 0)
    assert torch.allclose(plain.rms_norm(c, torch.ones(16, dtype=torch.float64), 0.0), torch.ones(1, 16, dtype=torch.float64))


# ---- rotary ------------------------------------------------------------------------------------
LLAMA3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 64}


def test_inv_freq_unscaled_and_factor_one():
    base = plain.rope_inv_freq(32, 10000.0)
    want = torch.tensor([10000.0 ** (-2 * i / 32) for i in range(16)])
    assert torch.allclose(base, want, rtol=1e-6)
    assert torch.equal(plain.rope_inv_freq(32, 10000.0, dict(LLAMA3, factor=1.0)), base)
    assert torch.equal(plain.rope_inv_freq(32, 10000.0, {"rope_type": "default", "factor": 8.0}), base)


def test_llama3_scaling_branches_and_continuity():
    base = plain.rope_inv_freq(32, 500000.0)
    scaled = plain.rope_inv_freq(32, 500000.0, LLAMA3)
    wavelen = 2 * math.pi / base
    short, long_ = wavelen < 16, wavelen > 64
    assert short.any() and long_.any() and (~short & ~long_).any()      # all three branches are hit
    assert torch.equal(scaled[short], base[short])                        # fast dims untouched
    assert torch.allclose(scaled[long_], base[long_] / 8.0, rtol=1e-6)    # slow dims divided by factor
    mid = ~short & ~long_
    assert ((scaled[mid] < base[mid]) & (scaled[mid] > base[mid] / 8.0)).all()


def _second_frequency_at_wavelength(inv_freq_fn, wavelen):
    """The function's own value, as a multiple of the unscaled frequency, for a frequency of exactly this
    wavelength: with two frequencies the second is theta^(-1/2), so theta = (wavelen / 2 pi)^2 puts it there."""
    theta = (wavelen / (2 * math.pi)) ** 2
    f = float(inv_freq_fn(4, theta)[1])
    assert math.isclose(2 * math.pi / f, wavelen, rel_tol=1e-6)
    return float(inv_freq_fn(4, theta, LLAMA3)[1]) / f


def _check_the_middle_band(inv_freq_fn):
    ratio = lambda wl: _second_frequency_at_wavelength(inv_freq_fn, wl)
    # hand values for factor 8, low 1, high 4, original 64: smooth = (64 / wl - 1) / 3 and the result is
    # ((1 - smooth) / 8 + smooth) f.  wl = 32: smooth 1/3 -> 5/12;  wl = 24: smooth 5/9 -> 11/18.
    assert math.isclose(ratio(32.0), 5 / 12, rel_tol=1e-6)      # swapped weights would give 17/24
    assert math.isclose(ratio(24.0), 11 / 18, rel_tol=1e-6)     # swapped: 37/72
    # the function is continuous at both ends of the band: just inside it agrees with the rule outside
    d = 1e-5
    assert ratio(16.0 * (1 - d)) == 1.0
    assert math.isclose(ratio(16.0 * (1 + d)), 1.0, rel_tol=2e-5)
    assert math.isclose(ratio(64.0 * (1 - d)), 1 / 8, rel_tol=1e-4)
    assert math.isclose(ratio(64.0 * (1 + d)), 1 / 8, rel_tol=1e-6)


def test_llama3_middle_band_by_hand_values_and_continuity_of_the_function():
    _check_the_middle_band(plain.rope_inv_freq)


def test_the_package_frequencies_obey_the_same_hand_values():
    from simple_inference_amd.parts.rope import rotary_inv_freq
    _check_the_middle_band(rotary_inv_freq)
    for dim, theta in ((32, 500000.0), (48, 25000.0)):
        assert torch.allclose(rotary_inv_freq(dim, theta, LLAMA3), plain.rope_inv_freq(dim, theta, LLAMA3), rtol=1e-6)


def test_rotation_pairs_i_with_i_plus_half():
    inv = plain.rope_inv_freq(8, 10000.0)
    cos, sin = plain.rope_tables(torch.tensor([3]), inv, torch.float64)
    x = torch.zeros(1, 1, 8, dtype=torch.float64)
    x[0, 0, 1] = 1.0
    y = plain.apply_rope(x, cos, sin)[0, 0]
    angle = 3 * inv[1].double()
    want = torch.zeros(8, dtype=torch.float64)
    want[1], want[5] = torch.cos(angle), torch.sin(angle)  # into element 1 + 4, with a plus sign; not into element 0 or 2
    assert torch.allclose(y, want, atol=1e-7)


def test_rotation_is_the_complex_product():
    D = 16
    inv = plain.rope_inv_freq(D, 10000.0).double()
    pos = torch.tensor([0, 1, 7, 100])
    cos, sin = plain.rope_tables(pos, inv.float(), torch.float64)
    x = torch.randn(4, 2, D, dtype=torch.float64)
    y = plain.apply_rope(x, cos, sin)
    z = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.polar(torch.ones(4, D // 2, dtype=torch.float64),
                                                                     torch.outer(pos.float(), inv.float()).double())[:, None, :]
    assert torch.allclose(y[..., :D // 2], z.real, atol=1e-6) and torch.allclose(y[..., D // 2:], z.imag, atol=1e-6)
    assert torch.equal(y[0], x[0])                                             # position 0 is the identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-9)            # a rotation keeps lengths


def test_rotated_dot_products_depend_on_distance_only():
    D = 32
    inv = plain.rope_inv_freq(D, 500000.0, LLAMA3)
    q, k = torch.randn(1, 1, D, dtype=torch.float64), torch.randn(1, 1, D, dtype=torch.float64)

    def dot(m, n):
        cq, sq = plain.rope_tables(torch.tensor([m]), inv, torch.float64)
        ck, sk = plain.rope_tables(torch.tensor([n]), inv, torch.float64)
        return float((plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum())
    assert math.isclose(dot(9, 4), dot(25, 20), rel_tol=1e-5, abs_tol=1e-5)
    assert not math.isclose(dot(9, 4), dot(4, 9), rel_tol=1e-3)   # the sign of the distance matters


# ---- attention ----------------------------------------------------------------------------------
def test_attention_without_mask_is_library_attention():
    q, k, v = torch.randn(5, 4, 16), torch.randn(9, 4, 16), torch.randn(9, 4, 16)
    out = plain.attention(q, k, v, torch.full((5,), 100), torch.arange(9))  # all keys visible
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-6)


def test_causal_grouped_attention_is_library_attention_on_repeated_heads():
    T, Hq, Hkv, D = 11, 6, 2, 8
    q, k, v = torch.randn(T, Hq, D), torch.randn(T, Hkv, D), torch.randn(T, Hkv, D)
    out = plain.attention(q, k, v, torch.arange(T), torch.arange(T))
    kr, vr = k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1)  # heads 0,1,2 read kv head 0
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1), is_causal=True)
    assert torch.allclose(out, ref.transpose(0, 1), atol=1e-6)


def test_attention_vector_of_the_reference_test():
    """serving/test_paged_kv_cache.py:160-179: seed 0, q [2,2,1,2], k,v [2,1,3,2], positions [[1],[2]],
    lengths [2,3]; masked attention equals library attention on each row's first ``length`` keys."""
    torch.manual_seed(0)
    q, k, v = torch.randn(2, 2, 1, 2), torch.randn(2, 1, 3, 2), torch.randn(2, 1, 3, 2)
    for b, (pos, length) in enumerate(((1, 2), (2, 3))):
        out = plain.attention(q[b].transpose(0, 1), k[b].transpose(0, 1), v[b].transpose(0, 1),
                              torch.tensor([pos]), torch.arange(3))
        ref = F.scaled_dot_product_attention(q[b:b + 1], k[b:b + 1, :, :length].repeat_interleave(2, dim=1),
                                             v[b:b + 1, :, :length].repeat_interleave(2, dim=1))
        assert torch.allclose(out.transpose(0, 1), ref[0], atol=1e-6)


def test_one_visible_key_gives_its_value_and_window_hides_old_keys():
    q, k, v = torch.randn(1, 2, 4), torch.randn(6, 1, 4), torch.randn(6, 1, 4)
    out = plain.attention(q, k, v, torch.tensor([0]), torch.arange(6))
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 1], v[0, 0])
    out = plain.attention(q, k, v, torch.tensor([5]), torch.arange(6), window=1)
    assert torch.allclose(out[0, 0], v[5, 0])
    a = plain.attention(q, k, v, torch.tensor([5]), torch.arange(6), window=3)
    b = plain.attention(q, k[3:], v[3:], torch.tensor([5]), torch.arange(3, 6))
    assert torch.allclose(a, b, atol=1e-6)


def test_scale_is_one_over_root_of_head_dim():
    q, k = torch.tensor([[[2.0, 0, 0, 0]]]), torch.tensor([[[1.0, 0, 0, 0]], [[0.0, 0, 0, 0]]])
    v = torch.tensor([[[1.0, 0, 0, 0]], [[0.0, 1, 0, 0]]])
    out = plain.attention(q, k, v, torch.tensor([1]), torch.arange(2))
    p = math.exp(2.0 / 2.0) / (math.exp(1.0) + 1.0)  # scores (2 * 1) / sqrt(4) and 0
    assert math.isclose(float(out[0, 0, 0]), p, rel_tol=1e-6)


# ---- feed-forward -------------------------------------------------------------------------------
def test_swiglu_is_silu_gate_times_up():
    x, wg, wu, wd = torch.randn(3, 8), torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    ref = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain.swiglu_mlp(x, wg, wu, wd), ref, atol=1e-6)
    assert torch.equal(plain.swiglu_mlp(x, torch.zeros(12, 8), wu, wd), torch.zeros(3, 8))  # silu(0) = 0


# ---- whole model --------------------------------------------------------------------------------
def tiny_model(seed=0, **over):
    cfg = {"hidden_size": 24, "intermediate_size": 40, "num_hidden_layers": 2, "vocab_size": 50,
           "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 8, "rms_norm_eps": 1e-5,
           "rope_theta": 10000.0, "rope_scaling": None, "tie_word_embeddings": True}
    cfg.update(over)
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.3
    H, I, D = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    w = {"model.embed_tokens.weight": r(cfg["vocab_size"], H), "model.norm.weight": 1 + r(H)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = 1 + r(H)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + r(H)
        w[f"{p}.self_attn.q_proj.weight"] = r(cfg["num_attention_heads"] * D, H)
        w[f"{p}.self_attn.k_proj.weight"] = r(cfg["num_key_value_heads"] * D, H)
        w[f"{p}.self_attn.v_proj.weight"] = r(cfg["num_key_value_heads"] * D, H)
        w[f"{p}.self_attn.o_proj.weight"] = r(H, cfg["num_attention_heads"] * D)
        w[f"{p}.mlp.gate_proj.weight"] = r(I, H)
        w[f"{p}.mlp.up_proj.weight"] = r(I, H)
        w[f"{p}.mlp.down_proj.weight"] = r(H, I)
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = r(cfg["vocab_size"], H)
    return cfg, w


def test_logits_do_not_change_when_all_positions_shift():
    """Only distances count: the same tokens at positions 17.. give the same logits as at 0..
    (fails if q and k are rotated differently, or values are rotated too)."""
    cfg, w = tiny_model()
    tokens = [3, 9, 9, 41, 0, 7]
    a = plain.forward(cfg, w, tokens, start_position=0)
    b = plain.forward(cfg, w, tokens, start_position=17)
    assert torch.allclose(a, b, atol=1e-5)


def test_logits_are_causal():
    cfg, w = tiny_model(seed=1)
    a = plain.forward(cfg, w, [5, 6, 7, 8])
    b = plain.forward(cfg, w, [5, 6, 7, 30])
    assert torch.allclose(a[:3], b[:3], atol=1e-12) and not torch.allclose(a[3], b[3])


def test_with_silent_layers_logits_are_head_of_norm_of_embedding():
    """Zero output projections leave the residual stream alone: the parts sit on side branches and
    the last norm and the (tied or untied) head follow the stream."""
    for tied in (True, False):
        cfg, w = tiny_model(seed=2, tie_word_embeddings=tied)
        for i in range(cfg["num_hidden_layers"]):
            w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
            w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
        tokens = [1, 2, 3]
        x = w["model.embed_tokens.weight"][tokens]
        head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
        want = F.rms_norm(x, (24,), w["model.norm.weight"], 1e-5) @ head.T
        assert torch.allclose(plain.forward(cfg, w, tokens), want, atol=1e-10)


def test_one_layer_by_hand():
    """One layer, one head, one token: attention returns v, so the block is two residual adds."""
    cfg, w = tiny_model(seed=3, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=24)
    t = [4]
    x = w["model.embed_tokens.weight"][t]
    n1 = F.rms_norm(x, (24,), w["model.layers.0.input_layernorm.weight"], 1e-5)
    x = x + (n1 @ w["model.layers.0.self_attn.v_proj.weight"].T) @ w["model.layers.0.self_attn.o_proj.weight"].T
    n2 = F.rms_norm(x, (24,), w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    x = x + plain.swiglu_mlp(n2, w["model.layers.0.mlp.gate_proj.weight"], w["model.layers.0.mlp.up_proj.weight"],
                             w["model.layers.0.mlp.down_proj.weight"])
    want = F.rms_norm(x, (24,), w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    assert torch.allclose(plain.forward(cfg, w, t), want, atol=1e-10)


# ---- sampling: the vectors of benchmarks/bench_sampling.py:42-129 -------------------------------------
def test_sampling_filters():
    torch.manual_seed(1)
    logits = torch.randn(8, 1000)
    kept = torch.isfinite(plain.filter_top_k(logits, 50))
    assert (kept.sum(-1) == 50).all()
    assert all(set(kept[i].nonzero().flatten().tolist()) == set(logits[i].topk(50).indices.tolist()) for i in range(8))
    assert torch.equal(plain.filter_top_k(logits, 0), logits) and torch.equal(plain.filter_top_k(logits, 1000), logits)
    assert torch.equal(plain.filter_top_p(logits, 1.0), logits)
    peaky = torch.full((16,), -1e4)
    peaky[7] = 0.0
    assert torch.isfinite(plain.filter_top_p(peaky, 0.5)).nonzero().flatten().tolist() == [7]
    torch.manual_seed(2)
    flat = 0.01 * torch.randn(1000)
    frac = torch.isfinite(plain.filter_top_p(flat, 0.5)).float().mean().item()
    assert 0.3 <= frac <= 0.7
    assert torch.isfinite(plain.filter_top_p(flat, 0.0)).sum() == 1


def test_sampling_by_inverse_cdf():
    torch.manual_seed(3)
    logits = torch.randn(200)
    assert plain.sample_with_uniform(logits, 0.3, temperature=0) == int(logits.argmax())
    probs = torch.softmax(logits.double(), -1)
    cdf = probs.cumsum(-1)
    for u in (0.0, 0.1, 0.5, 0.999):
        t = plain.sample_with_uniform(logits, u, temperature=1.0)
        assert (cdf[t - 1] if t else 0.0) <= u < cdf[t] + 1e-12
    # the frequencies of many draws follow the probabilities
    g = torch.Generator().manual_seed(4)
    small = torch.tensor([0.0, 1.0, 2.0, -1.0])
    counts = torch.zeros(4)
    for u in torch.rand(4000, generator=g).tolist():
        counts[plain.sample_with_uniform(small, u, temperature=0.7)] += 1
    assert torch.allclose(counts / 4000, torch.softmax(small / 0.7, -1), atol=0.03)
    only = plain.sample_with_uniform(small, 0.9, temperature=1.0, top_k=1)
    assert only == 2


def test_the_model_with_the_references_roundings_is_the_model_when_nothing_is_rounded(tmp_path):
    """``forward_as_the_reference_rounds`` composes the same part functions; with a rounding that does nothing it is
    ``forward``, and with bfloat16 roundings it lies near it, further for more layers."""
    from helpers import TINIES, random_tokens, rel_err, write_tiny_model
    import copy
    tiny = TINIES["b"]
    folder = write_tiny_model(tmp_path / "b", tiny, seed=3)
    cfg, w = plain.read_model(folder, torch.float64)
    tokens = random_tokens(cfg["vocab_size"], 40, seed=1)
    exact = plain.forward(cfg, w, tokens)
    same = plain.forward_as_the_reference_rounds(cfg, w, tokens, rnd=lambda t: t)
    assert torch.equal(same, exact)
    rows = plain.forward_as_the_reference_rounds(cfg, w, tokens, rows=[3, 39], rnd=lambda t: t)
    assert torch.allclose(rows, exact[[3, 39]], rtol=0, atol=1e-12)     # a product of 2 rows sums in another order
    rounded = plain.forward_as_the_reference_rounds(cfg, w, tokens)
    assert 1e-4 < rel_err(rounded, exact) < 2.5e-2
    deep = copy.deepcopy(tiny.config)
    deep["num_hidden_layers"] = 12
    folder = write_tiny_model(tmp_path / "deep", tiny, seed=3, config=deep)
    cfg12, w12 = plain.read_model(folder, torch.float64)
    exact12 = plain.forward(cfg12, w12, tokens)
    assert rel_err(plain.forward_as_the_reference_rounds(cfg12, w12, tokens), exact12) > rel_err(rounded, exact)
