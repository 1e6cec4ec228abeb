"""Typed engine configuration.

The names and meanings follow the keyword arguments of the reference's
``InferenceEngine`` (``serving/engine.py:96-113``) where it has them:
``max_running``, ``max_seq_len``, ``block_size``, ``num_kv_blocks``,
``token_budget``, ``eos_id``, ``warmup``, ``use_prefix_cache`` and
``prefix_cache_blocks`` mean what they mean there; ``use_graphs`` is its
``use_cuda_graphs`` (hipGraph here).  ``profile_ranges`` switches on the named
ranges that the reference always records (``serving/engine.py:334,342,359``).  ``chunk_tokens``, ``dtype``
and ``run_ahead`` have no counterpart there: the reference prefills whole prompts (``plan.md:811-868``
only sketches portions) and has no 32-bit GPU path.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32,
}


def resolve_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name)]
    except KeyError:
        raise ValueError(f"engine dtype must be one of {sorted(_DTYPES)}, got {name!r}") from None


@dataclass
class EngineConfig:
    max_running: int = 8                  # concurrent requests (state slots)
    max_seq_len: int = 4096               # prompt + generated tokens of one request
    block_size: int = 16                  # tokens per cache page
    num_kv_blocks: Optional[int] = None   # pages per layer group; None → max_running * pages(max_seq_len)
    token_budget: Optional[int] = None    # cap on the context admitted at once; None → max_running * max_seq_len
    chunk_tokens: int = 512               # most tokens one step runs (decoded tokens + prompt portions)
    dtype: str = "bfloat16"               # "bfloat16" (serving kernels) or "float32" (true 32-bit everywhere)
    eos_id: Optional[int] = None          # None → the model configuration's; -1 → never stop on a token
    use_graphs: Optional[bool] = None     # replay decode-only steps from captured hipGraphs; None → on a GPU, yes
    run_ahead: bool = True                # with graphs: launch the next decode step before this one's tokens are read
    use_prefix_cache: bool = False        # reuse complete pages of equal prompt prefixes
    prefix_cache_blocks: Optional[int] = None
    warmup: bool = False
    profile_ranges: bool = False          # named ranges (profiler, roctx) around schedule / forward / sample / collect
    device: str = "cuda:0"

    def __post_init__(self):
        if self.max_running <= 0:
            raise ValueError(f"max_running must be positive, got {self.max_running}")
        if self.max_seq_len <= 0:
            raise ValueError(f"max_seq_len must be positive, got {self.max_seq_len}")
        if self.block_size <= 0 or self.block_size & (self.block_size - 1):
            raise ValueError(f"block_size must be a positive power of two, got {self.block_size}")
        if self.chunk_tokens <= 0:
            raise ValueError(f"chunk_tokens must be positive, got {self.chunk_tokens}")
        if self.num_kv_blocks is not None and self.num_kv_blocks <= 0:
            raise ValueError(f"num_kv_blocks must be positive, got {self.num_kv_blocks}")
        resolve_dtype(self.dtype)

    @property
    def torch_dtype(self) -> torch.dtype:
        return resolve_dtype(self.dtype)

    def graphs_wanted(self) -> bool:
        if self.use_graphs is not None:
            return bool(self.use_graphs)
        return torch.device(self.device).type == "cuda"

    def pages_per_request(self) -> int:
        return -(-self.max_seq_len // self.block_size)

    def resolved_num_kv_blocks(self) -> int:
        if self.num_kv_blocks is not None:
            return self.num_kv_blocks
        return self.max_running * self.pages_per_request()

    def resolved_token_budget(self) -> int:
        if self.token_budget is not None:
            return self.token_budget
        return self.max_running * self.max_seq_len
