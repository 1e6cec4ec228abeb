"""Seeded random weights: in memory, or written as a model folder.

The reference has random weights only inside a test (``serving/test_paged_kv_cache.py:204-207``:
``normal_(p, 0, 0.02)`` over every parameter).  Here it is a mode of its own: every
tensor the model's parts want is drawn in the plan's fixed order from one generator:
matrices ``N(0, std)``, norm gains ``1 + N(0, gain_std)``.  ``write_model_folder``
stores them with ``config.json`` so that any program that reads a model folder can
read this one.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Mapping

import torch

from ..parts.plan import TensorSpec

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def random_tensors(expected: Mapping[str, TensorSpec], seed: int, std: float = 0.02, gain_std: float = 0.0,
                   storage: str = "bfloat16", device="cpu") -> Dict[str, torch.Tensor]:
    """One tensor per expected name, in storage dtype (vectors and matrices alike)."""
    dtype = _STORAGE[storage]
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        if spec.role == "table":
            raise ValueError(f"no random rule for integer table {name}")
        t = torch.empty(spec.shape, dtype=torch.float32, device=device)
        if spec.role == "vector":
            t.normal_(0.0, 1.0, generator=gen).mul_(gain_std).add_(1.0)
        else:
            t.normal_(0.0, std, generator=gen)
        out[name] = t.to(dtype)
    return out


def write_model_folder(folder, config_dict: Mapping, tensors: Mapping[str, torch.Tensor]) -> Path:
    """Writes ``config.json`` and ``model.safetensors``."""
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    with open(folder / "config.json", "w") as f:
        json.dump(dict(config_dict), f, indent=2)
    save_file({k: v.detach().cpu().contiguous() for k, v in tensors.items()},
              str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder
