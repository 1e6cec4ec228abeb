"""Seeded random configurations of the architecture through trace replay on the GPU, against the plain
implementation: head sizes in steps of 16, any number of heads and groups, widths and vocabularies that are
no multiple of anything convenient beside widths in multiples of 64 (which steps of few tokens run through the
products with fused epilogues), every option on and off."""

import random

import pytest
import torch

from helpers import TOLERANCE, Tiny, plain_logits, rel_err, write_tiny_model
from test_trace_run import collect, make_trace

pytestmark = pytest.mark.gpu

HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 256)   # the head sizes whose attention kernels are built beforehand


def random_config(seed):
    rng = random.Random(seed)
    head_dim = HEAD_DIMS[seed % len(HEAD_DIMS)]
    n_kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 7])
    scaling = None
    if rng.random() < 0.6:
        scaling = {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0, 32.0]), "low_freq_factor": 1.0,
                   "high_freq_factor": rng.choice([2.0, 4.0]),
                   "original_max_position_embeddings": rng.choice([16, 64, 256])}
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": rng.choice([40, 72, 100, 128, 136, 192, 200, 264, 320]),
        "intermediate_size": rng.choice([56, 96, 150, 192, 224, 256, 328]),
        "num_hidden_layers": rng.choice([1, 2, 3]), "vocab_size": rng.choice([97, 257, 500, 1001]),
        "num_attention_heads": n_kv * group, "num_key_value_heads": n_kv, "head_dim": head_dim,
        "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-4]), "rope_theta": rng.choice([10000.0, 500000.0]),
        "rope_scaling": scaling, "max_position_embeddings": 1024, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": rng.random() < 0.5, "torch_dtype": "bfloat16", "hidden_act": "silu",
    }


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(9))
def test_random_configuration_replays_like_the_plain_implementation(tmp_path, seed, dtype):
    from simple_inference_amd.replay import TraceReplayer

    cfg = random_config(seed)
    print("configuration", seed, {k: cfg[k] for k in ("hidden_size", "intermediate_size", "num_hidden_layers",
          "vocab_size", "num_attention_heads", "num_key_value_heads", "head_dim", "tie_word_embeddings")}, flush=True)
    folder = write_tiny_model(tmp_path, Tiny(f"r{seed}", cfg, 16, 0.05, 0.1), seed=300 + seed)
    steps, prompts, most = make_trace(cfg["vocab_size"], lengths=(50, 33, 71, 20, 64))
    page = (8, 16, 32, 64)[seed % 4]
    rp = TraceReplayer(folder, dtype, most, block_size=page)
    got = collect(steps, lambda st: rp.step(st["entries"], st["end"]).float().cpu().numpy())
    tol = TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"]
    for r, toks in prompts.items():
        ref = plain_logits(folder, toks)
        mine = torch.stack([torch.as_tensor(got[r][p]) for p in range(len(toks))])
        assert rel_err(mine, ref) <= tol, (r, rel_err(mine, ref))
    assert rp.cache.free_pages() == -(-most // page) and not rp.ids
