"""From a model folder (or a configuration and a seed) to a model with its weights bound."""

from __future__ import annotations

from typing import Mapping

import torch

from ..config.engine_config import EngineConfig
from ..config.model_config import read_config_json
from ..config.registry import architecture_of
from ..parts.context import BuildEnv
from ..parts.model import DecoderModel
from ..weights.loader import load_weights, target_dtype
from ..weights.random_init import random_tensors


def default_kernels():
    """The compiled HIP kernel library; raises if it cannot be had."""
    from ..kernels import HipKernels
    return HipKernels()


def build_model(config_dict: Mapping, engine_cfg: EngineConfig, kernels):
    """(model without weights, the architecture's typed configuration)."""
    arch = architecture_of(config_dict)
    model_cfg = arch.parse_config(config_dict)
    plan = arch.build_plan(model_cfg)
    max_positions = engine_cfg.max_seq_len
    if plan.max_position_embeddings is not None and max_positions > plan.max_position_embeddings:
        raise ValueError(
            f"max_seq_len {max_positions} exceeds the model's max_position_embeddings "
            f"{plan.max_position_embeddings}")
    env = BuildEnv(kernels=kernels, device=torch.device(engine_cfg.device), dtype=engine_cfg.torch_dtype,
                   max_positions=max_positions)
    return DecoderModel(plan, env), model_cfg


def model_from_folder(folder, engine_cfg: EngineConfig, kernels=None):
    kernels = kernels if kernels is not None else default_kernels()
    model, model_cfg = build_model(read_config_json(folder), engine_cfg, kernels)
    tensors = load_weights(folder, model.expected_tensors(), engine_cfg.device, engine_cfg.torch_dtype)
    model.bind(tensors)
    return model, model_cfg


def model_from_random(config_dict: Mapping, seed: int, engine_cfg: EngineConfig, kernels=None,
                      std: float = 0.02, gain_std: float = 0.0, storage: str = "bfloat16",
                      generate_on_device: bool = False):
    """Random weights without a folder.  Values are drawn in ``storage`` dtype first, so
    that a bfloat16 and a float32 engine built from the same seed hold the same numbers."""
    kernels = kernels if kernels is not None else default_kernels()
    model, model_cfg = build_model(config_dict, engine_cfg, kernels)
    expected = model.expected_tensors()
    device = engine_cfg.device if generate_on_device else "cpu"
    drawn = random_tensors(expected, seed, std, gain_std, storage, device=device)
    tensors = {
        name: t.to(device=engine_cfg.device,
                   dtype=target_dtype(t.dtype, expected[name].role, engine_cfg.torch_dtype)).contiguous()
        for name, t in drawn.items()
    }
    model.bind(tensors)
    return model, model_cfg
