"""Named config.json dictionaries: data, not code paths.

These are the shapes that the measurement program and the command line can
build random weights for.  Each is the dictionary a config.json of that model
would hold, and goes through the same ``parse_config`` as a file does.  The
reference has one preset, ``ModelConfig.llama_3_2_3b`` (``config.py:111-135``).
"""

from __future__ import annotations

import copy

_LLAMA3_SCALING_32 = {
    "rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
    "high_freq_factor": 4.0, "original_max_position_embeddings": 8192,
}

PRESETS = {
    "llama-3.2-3b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 3072, "intermediate_size": 8192, "num_hidden_layers": 28,
        "vocab_size": 128256, "num_attention_heads": 24, "num_key_value_heads": 8, "head_dim": 128,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "rope_scaling": _LLAMA3_SCALING_32,
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "llama-3.2-1b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 2048, "intermediate_size": 8192, "num_hidden_layers": 16,
        "vocab_size": 128256, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "rope_scaling": _LLAMA3_SCALING_32,
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "llama-3.1-8b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 4096, "intermediate_size": 14336, "num_hidden_layers": 32,
        "vocab_size": 128256, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
        "rope_scaling": dict(_LLAMA3_SCALING_32, factor=8.0),
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "tiny-a": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2,
        "vocab_size": 256, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
        "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
        "max_position_embeddings": 2048, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "tiny-b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 96, "intermediate_size": 224, "num_hidden_layers": 3,
        "vocab_size": 384, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
        "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                         "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
        "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
}


def preset(name: str) -> dict:
    try:
        return copy.deepcopy(PRESETS[name])
    except KeyError:
        raise KeyError(f"unknown preset {name!r}; known: {', '.join(sorted(PRESETS))}") from None
