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


def count_parameters(model, model_cfg) -> int:
    """Elements over all tensors the parts ask for (a shared tensor once).  Where the architecture's configuration
    has a formula of its own for the count (reference: ``loader.py:301-316`` checks the total it loaded against
    the known size of the model) the two must agree: the parts' shapes and the formula are written from the same
    config.json keys by different code."""
    total = 0
    for spec in model.expected_tensors().values():
        n = 1
        for d in spec.shape:
            n *= d
        total += n
    formula = getattr(model_cfg, "num_parameters", None)
    if formula is not None and formula() != total:
        raise ValueError(f"the model's parts hold {total:,} parameters, the configuration's formula says {formula():,}")
    return total


def describe(model, model_cfg, engine_cfg: EngineConfig) -> str:
    """One line: architecture, parameters, bytes of the cache a token (reference: ``loader.py:301-316``,
    ``config.py:144-149`` print the same two figures)."""
    el = 2 if engine_cfg.dtype == "bfloat16" else 4
    kv = sum(need.num_kv_heads * (need.head_dim + need.value_dim) * slabs * el
             for need, slabs in zip(model.cache_layout().kv_groups, model.cache_layout().kv_slabs))
    name = getattr(model_cfg, "architecture", type(model_cfg).__name__)
    return (f"{name}: {count_parameters(model, model_cfg):,} parameters in {len(model.order)} layers, "
            f"{kv:,} bytes of cache a token ({engine_cfg.dtype})")


def model_from_folder(folder, engine_cfg: EngineConfig, kernels=None):
    kernels = kernels if kernels is not None else default_kernels()
    model, model_cfg = build_model(read_config_json(folder), engine_cfg, kernels)
    count_parameters(model, model_cfg)
    tensors = load_weights(folder, model.expected_tensors(), engine_cfg.device, engine_cfg.torch_dtype,
                           duplicates=model.plan.duplicates)
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
