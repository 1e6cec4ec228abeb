"""Shared pieces of the tests: tiny configurations, model folders, engines, traces."""

from __future__ import annotations

import copy
import os
from dataclasses import dataclass

import torch

import plain_llama as plain

# Three tiny configurations that differ in every size and option.  A: 2 layers, 4 query / 2 key-value
# heads of 16, tied head, no frequency scaling, pages of 4.  B: 3 layers, 3 / 1 heads of 32, untied head,
# llama3 scaling, pages of 8.  C has sizes that are no power of two, a head size that is not
# hidden / heads, as many key/value heads as query heads, and another scaling.  D has widths in multiples of
# 64 and heads of 64: the sizes at which steps of few tokens take the products that rotate and write the cache,
# add into the residual and share out the norm between them.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2, "vocab_size": 256,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 2048, "bos_token_id": 1, "eos_token_id": 2,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 96, "intermediate_size": 224, "num_hidden_layers": 3, "vocab_size": 384,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 2,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
}
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 120, "intermediate_size": 200, "num_hidden_layers": 2, "vocab_size": 331,
    "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 48,
    "rms_norm_eps": 3e-5, "rope_theta": 25000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 2.0, "original_max_position_embeddings": 32},
    "max_position_embeddings": 1024, "bos_token_id": 0, "eos_token_id": 5,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
}
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 128, "intermediate_size": 192, "num_hidden_layers": 3, "vocab_size": 320,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 64,
    "rms_norm_eps": 2e-6, "rope_theta": 100000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 2.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 3.0, "original_max_position_embeddings": 48},
    "max_position_embeddings": 2048, "bos_token_id": 3, "eos_token_id": 4,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
}


@dataclass
class Tiny:
    name: str
    config: dict
    page_size: int
    std: float
    gain_std: float


TINIES = {
    "a": Tiny("a", TINY_A, 4, 0.02, 0.1),
    "b": Tiny("b", TINY_B, 8, 0.05, 0.0),
    "c": Tiny("c", TINY_C, 16, 0.04, 0.2),
    "d": Tiny("d", TINY_D, 16, 0.06, 0.15),
}


def write_tiny_model(folder, tiny: Tiny, seed: int = 0, storage: str = "bfloat16", config=None):
    """Writes config.json + model.safetensors with the package's random-weights mode."""
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    from simple_inference_amd.weights import random_tensors, write_model_folder

    cfg = copy.deepcopy(config if config is not None else tiny.config)
    model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    tensors = random_tensors(model.expected_tensors(), seed, tiny.std, tiny.gain_std, storage)
    write_model_folder(folder, mcfg.to_dict(), tensors)
    return folder


def random_tokens(vocab: int, n: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def make_runner(folder, backend: str, page_size: int, num_pages: int, max_seq_len: int = 512, max_running: int = 4):
    """(StepRunner, CacheManager, model config) on one of: 'twins' (CPU), 'hip-f32', 'hip-bf16'."""
    from simple_inference_amd.cache import CacheManager
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import StepRunner, model_from_folder

    if backend == "twins":
        from twins import TwinKernels
        kernels, device, dtype = TwinKernels(), "cpu", "float32"
    else:
        from simple_inference_amd.kernels import HipKernels
        kernels, device = HipKernels(), "cuda:0"
        dtype = {"hip-f32": "float32", "hip-bf16": "bfloat16"}[backend]
    ecfg = EngineConfig(device=device, dtype=dtype, max_seq_len=max_seq_len, block_size=page_size,
                        num_kv_blocks=num_pages, max_running=max_running)
    model, mcfg = model_from_folder(folder, ecfg, kernels)
    cache = CacheManager(model.cache_layout(), page_size=page_size, num_pages=num_pages, max_running=max_running,
                         dtype=ecfg.torch_dtype, device=device)
    return StepRunner(model, cache, kernels, device, max_seq_len), cache, mcfg


def plain_logits(folder, tokens):
    cfg, w = plain.read_model(folder)
    return plain.forward(cfg, w, tokens)


# Differences are measured against the size of the logits: max |a - b| / max |b|.
# float32: the engine and the plain implementation differ by the order of float additions only.
# bfloat16: activations carry 8 bits of mantissa (2^-9 relative rounding) through every layer.
TOLERANCE = {"twins": 2e-5, "hip-f32": 2e-5, "hip-bf16": 2.5e-2}


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


BACKENDS_ENV = os.environ.get("SIA_TEST_BACKENDS")
