"""A plain, slow implementation of the Llama decoder, written from the reference's formulas.

Whole sequences, no cache, float32 (or float64), one function for each part.  It
shares no code with the engine: it reads config.json and the safetensors file
itself and uses only elementary torch operations.  Every function cites the lines
of the reference whose formula it writes down.  The reference
is read, not run.

Where the reference has two variants of one formula that differ only in where they
round to bfloat16 (a PyTorch path and a fused kernel path), this file computes the
unrounded mathematical value, which both approximate.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# ---------------------------------------------------------------------------
# configuration and weights
# ---------------------------------------------------------------------------

def read_config(folder):
    with open(Path(folder) / "config.json") as f:
        return json.load(f)


def read_model(folder, dtype=torch.float32):
    """(config dict, {tensor name: tensor}) of a model folder."""
    from safetensors.torch import load_file

    folder = Path(folder)
    cfg = read_config(folder)
    tensors = {k: v.to(dtype) for k, v in load_file(str(folder / "model.safetensors")).items()}
    return cfg, tensors


def head_dim_of(cfg) -> int:
    # reference: config.py:81 derives hidden_size // num_attention_heads; a config.json
    # that states head_dim is taken at its word.
    return int(cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"])


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------

def rms_norm(x, weight, eps):
    """reference: ops/rmsnorm.py:41-46 — x * rsqrt(mean(x^2) + eps) * w; eps inside the root."""
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight


def rope_inv_freq(head_dim, theta, scaling=None):
    """reference: ops/rope.py:95-97 (base) and ops/rope.py:120-155 (llama3 scaling).

    The base frequencies are computed in float32 and the scaling loop runs in Python
    floats over them, as there.
    """
    idx = torch.arange(0, head_dim, 2, dtype=torch.float32)
    freqs = 1.0 / (theta ** (idx / head_dim))
    if not scaling or scaling.get("rope_type", scaling.get("type", "default")) != "llama3":
        return freqs
    factor = float(scaling.get("factor", 1.0))
    low = float(scaling.get("low_freq_factor", 1.0))
    high = float(scaling.get("high_freq_factor", 4.0))
    orig = float(scaling.get("original_max_position_embeddings", 8192))
    low_freq_wavelen = orig / low
    high_freq_wavelen = orig / high
    out = []
    for f in freqs.tolist():
        wavelen = 2 * math.pi / f
        if wavelen < high_freq_wavelen:
            out.append(f)
        elif wavelen > low_freq_wavelen:
            out.append(f / factor)
        else:
            smooth = (orig / wavelen - low) / (high - low)
            out.append((1 - smooth) * f / factor + smooth * f)
    return torch.tensor(out, dtype=torch.float32)


def rope_tables(positions, inv_freq, dtype=torch.float32):
    """reference: ops/rope.py:108-118 — angles = outer(float32 positions, freqs), duplicated
    over both halves; cos and sin of them (float32 there)."""
    angles = torch.outer(positions.to(torch.float32), inv_freq)
    angles = torch.cat([angles, angles], dim=-1)
    return angles.cos().to(dtype), angles.sin().to(dtype)


def rotate_half(x):
    """reference: ops/rope.py:167-182 — [x1, x2] -> [-x2, x1] over the two halves."""
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rope(x, cos, sin):
    """reference: ops/rope.py:212-213 — x * cos + rotate_half(x) * sin; x is [T, heads, D]."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def attention(q, k, v, q_positions, k_positions, scale=None, window=None, rnd=None):
    """Scores, mask, softmax, weighted sum.

    q [Tq, Hq, D]; k, v [Tk, Hkv, D].  reference: kernels/attention_kernel.py:184-251 —
    query head h reads kv head h // (Hq // Hkv); S = (q . k) * scale with
    scale = 1 / sqrt(D) applied after the dot; key j visible iff position(j) <= position(query)
    (serving/paged_kv_cache.py:366-375 writes the same mask explicitly); softmax over the
    visible keys; O = P V.  ``window`` w additionally hides keys at distance >= w.  ``rnd`` (see
    ``forward_as_the_reference_rounds``) is applied to the probabilities before P V
    (kernels/attention_kernel.py:241 casts p to the values' dtype).
    """
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    group = Hq // Hkv
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    out = torch.empty_like(q)
    visible = k_positions[None, :] <= q_positions[:, None]
    if window is not None:
        visible &= k_positions[None, :] > (q_positions[:, None] - window)
    for h in range(Hq):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.T) * scale
        scores = scores.masked_fill(~visible, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        if rnd is not None:
            # the kernel rounds exp(s - m) before P V and divides the float sum at the end; rounding the
            # normalised probabilities instead differs by the rounding of one common factor
            probs = rnd(probs)
        out[:, h, :] = probs @ vh
    return out


def swiglu_mlp(x, w_gate, w_up, w_down):
    """reference: ops/mlp.py:117-128 — down(silu(gate(x)) * up(x)); silu(g) = g * sigmoid(g)."""
    g = x @ w_gate.T
    u = x @ w_up.T
    return ((g * torch.sigmoid(g)) * u) @ w_down.T


def attention_layer(x, positions, w, prefix, cfg, inv_freq):
    """reference: ops/attention.py:128-226 — project, view as heads, rotate q and k, attend, project."""
    T = x.shape[0]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim_of(cfg)
    q = (x @ w[f"{prefix}.self_attn.q_proj.weight"].T).view(T, Hq, D)
    k = (x @ w[f"{prefix}.self_attn.k_proj.weight"].T).view(T, Hkv, D)
    v = (x @ w[f"{prefix}.self_attn.v_proj.weight"].T).view(T, Hkv, D)
    cos, sin = rope_tables(positions, inv_freq, x.dtype)
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    o = attention(q, k, v, positions, positions)
    return o.reshape(T, Hq * D) @ w[f"{prefix}.self_attn.o_proj.weight"].T


def block(x, positions, w, i, cfg, inv_freq):
    """reference: model/block.py:135-147 — x += attn(norm1(x)); x += mlp(norm2(x))."""
    p = f"model.layers.{i}"
    eps = cfg["rms_norm_eps"]
    x = x + attention_layer(rms_norm(x, w[f"{p}.input_layernorm.weight"], eps), positions, w, p, cfg, inv_freq)
    x = x + swiglu_mlp(rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps),
                       w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                       w[f"{p}.mlp.down_proj.weight"])
    return x


def forward(cfg, w, tokens, start_position=0, rows=None):
    """Logits [T, V] of one whole sequence (with ``rows``: at those places only, [len(rows), V]; the layers
    still see the whole sequence).  reference: model/llama.py:173-186 —
    embed -> blocks -> norm -> head; tied head = embedding matrix (ops/embedding.py:84-92)."""
    device = w["model.embed_tokens.weight"].device      # the weights may lie on a GPU: then so does everything
    tokens = torch.as_tensor(tokens, dtype=torch.long, device=device)
    positions = torch.arange(start_position, start_position + len(tokens), device=device)
    inv_freq = rope_inv_freq(head_dim_of(cfg), float(cfg["rope_theta"]), cfg.get("rope_scaling")).to(device)
    x = w["model.embed_tokens.weight"][tokens]
    for i in range(cfg["num_hidden_layers"]):
        x = block(x, positions, w, i, cfg, inv_freq)
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long, device=device)]
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", True) else w["lm_head.weight"]
    return x @ head.T


# ---------------------------------------------------------------------------
# the same model with the reference's bfloat16 roundings
# ---------------------------------------------------------------------------

def to_bfloat16_and_back(t):
    return t.to(torch.bfloat16).to(t.dtype)


def forward_as_the_reference_rounds(cfg, w, tokens, rows=None, rnd=to_bfloat16_and_back):
    """``forward`` with every intermediate result rounded where the reference's bfloat16 model materialises a
    bfloat16 tensor on its production path (the fused kernels: one rounding each).  Computed in the weights' dtype
    (float64 for a yardstick) apart from those roundings, it shows how far a *correct* bfloat16 implementation of
    this model lies from exact arithmetic on given weights and tokens: the measure for what a bfloat16 engine may
    differ by.  Places, in the order of a block (model/block.py:135-147):

    * the norm's output (kernels/rmsnorm_kernel.py:105-113: float statistics and gain, one rounding);
    * q, k, v as the products leave the BLAS library (ops/attention.py:128-130);
    * the cos/sin rows, cast to the activations' dtype (ops/attention.py:143-145), and the rotated q and k
      (kernels/rope_kernel.py:131-154: float arithmetic, one rounding);
    * the probabilities before P V (kernels/attention_kernel.py:241) and the attention's output (:250);
    * the output projection (ops/attention.py:226) and the residual sum, which the reference keeps in the
      activations' dtype (model/block.py:139);
    * gate and up (ops/mlp.py:117), silu(gate) * up (kernels/swiglu_kernel.py:142-150: float, one rounding),
      the down projection (ops/mlp.py:128) and the second residual sum (model/block.py:145);
    * the last norm (model/llama.py:181).  The logits are left as the exact product of that rounded row: the
      reference rounds them too (model/llama.py:184), which a bound should not profit from.
    """
    device = w["model.embed_tokens.weight"].device
    tokens = torch.as_tensor(tokens, dtype=torch.long, device=device)
    T = len(tokens)
    positions = torch.arange(T, device=device)
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim_of(cfg)
    eps = cfg["rms_norm_eps"]
    inv_freq = rope_inv_freq(D, float(cfg["rope_theta"]), cfg.get("rope_scaling")).to(device)
    x = w["model.embed_tokens.weight"][tokens]
    cos, sin = rope_tables(positions, inv_freq, x.dtype)
    cos, sin = rnd(cos), rnd(sin)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        h = rnd(rms_norm(x, w[f"{p}.input_layernorm.weight"], eps))
        q = rnd(h @ w[f"{p}.self_attn.q_proj.weight"].T).view(T, Hq, D)
        k = rnd(h @ w[f"{p}.self_attn.k_proj.weight"].T).view(T, Hkv, D)
        v = rnd(h @ w[f"{p}.self_attn.v_proj.weight"].T).view(T, Hkv, D)
        q, k = rnd(apply_rope(q, cos, sin)), rnd(apply_rope(k, cos, sin))
        o = rnd(attention(q, k, v, positions, positions, rnd=rnd))
        x = rnd(x + rnd(o.reshape(T, Hq * D) @ w[f"{p}.self_attn.o_proj.weight"].T))
        h = rnd(rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps))
        g = rnd(h @ w[f"{p}.mlp.gate_proj.weight"].T)
        u = rnd(h @ w[f"{p}.mlp.up_proj.weight"].T)
        a = rnd((g * torch.sigmoid(g)) * u)
        x = rnd(x + rnd(a @ w[f"{p}.mlp.down_proj.weight"].T))
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long, device=device)]
    x = rnd(rms_norm(x, w["model.norm.weight"], eps))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", True) else w["lm_head.weight"]
    return x @ head.T


# ---------------------------------------------------------------------------
# sampling (reference: sampling.py:40-173)
# ---------------------------------------------------------------------------

def filter_top_k(logits, k):
    """reference: sampling.py:69-84 — below the k-th largest value -> -inf; ties with it stay."""
    V = logits.shape[-1]
    if k <= 0 or k >= V:
        return logits
    kth = torch.sort(logits, descending=True).values[..., k - 1:k]
    return torch.where(logits < kth, torch.full_like(logits, float("-inf")), logits)


def filter_top_p(logits, p):
    """reference: sampling.py:96-129 — sort descending, softmax, cumulative sum; a token goes
    iff the mass of the tokens before it already exceeds p (so the one that crosses p stays)."""
    if p >= 1.0:
        return logits
    if p <= 0.0:
        return filter_top_k(logits, 1)
    sorted_logits, idx = torch.sort(logits, descending=True, dim=-1)
    cum = torch.softmax(sorted_logits, dim=-1).cumsum(dim=-1)
    remove_sorted = torch.zeros_like(cum, dtype=torch.bool)
    remove_sorted[..., 1:] = cum[..., :-1] > p
    remove = torch.zeros_like(remove_sorted).scatter(-1, idx, remove_sorted)
    return logits.masked_fill(remove, float("-inf"))


def filtered_probs(logits, temperature=1.0, top_k=0, top_p=1.0):
    """reference: sampling.py:141-172 — /T, then top-k, then top-p, then softmax in float32+."""
    logits = logits.to(torch.float64) / temperature
    if top_k > 0:
        logits = filter_top_k(logits, top_k)
    if top_p < 1.0:
        logits = filter_top_p(logits, top_p)
    return torch.softmax(logits, dim=-1)


def sample_with_uniform(logits, u, temperature=1.0, top_k=0, top_p=1.0):
    """temperature == 0 -> argmax (sampling.py:160-161).  Otherwise the reference draws with
    torch.multinomial from the global generator (sampling.py:173), which cannot be replayed;
    the engine instead inverts the cumulative distribution at a given uniform ``u``: the token
    is the first whose cumulative probability exceeds u."""
    if temperature == 0:
        return int(torch.argmax(logits))
    cdf = filtered_probs(logits, temperature, top_k, top_p).cumsum(-1)
    return int(min(int((cdf <= u * cdf[-1]).sum()), logits.shape[-1] - 1))
