"""Drives the engine's own model, step function, cache manager and kernels from a trace.

A trace names, step by step, which requests bring which tokens.  The scheduler and the
sampler stay out of it: the tokens are given.  A request is admitted to the cache when it
first appears (no pages are promised, since its length is not known; pages are taken as it
grows) and its pages and slot go back when the trace ends it.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .cache.manager import CacheManager
from .config.engine_config import EngineConfig
from .config.model_config import read_config_json
from .engine.build import default_kernels, model_from_folder
from .engine.step import StepEntry, StepRunner


class TraceReplayer:
    def __init__(self, model_folder, dtype: str, max_tokens: int, block_size: Optional[int] = None,
                 max_live: int = 8, device: str = "cuda:0", kernels=None):
        cfg = read_config_json(model_folder)
        defaults = EngineConfig()
        page = block_size or defaults.block_size
        if 64 % page and page % 64:
            raise ValueError(f"block_size {page} neither divides 64 nor is a multiple of it")
        num_pages = max(1, -(-max_tokens // page))
        max_pos = int(cfg.get("max_position_embeddings", max_tokens))
        self.engine_cfg = EngineConfig(
            device=device, dtype=dtype, block_size=page, num_kv_blocks=num_pages, max_running=max_live,
            max_seq_len=min(max_pos, max(max_tokens, page)))
        self.kernels = kernels if kernels is not None else default_kernels()
        self.architecture = (cfg.get("architectures") or ["?"])[0]
        self.model, self.model_cfg = model_from_folder(model_folder, self.engine_cfg, self.kernels)
        self.cache = CacheManager(
            self.model.cache_layout(), page_size=page, num_pages=num_pages, max_running=max_live,
            dtype=self.engine_cfg.torch_dtype, device=device)
        self.runner = StepRunner(self.model, self.cache, self.kernels, device, self.engine_cfg.max_seq_len)
        self.ids: Dict[str, int] = {}
        self._next = 1

    def describe(self) -> str:
        return (f"{self.architecture}, dtype {self.engine_cfg.dtype}, {self.engine_cfg.num_kv_blocks} "
                f"pages of {self.engine_cfg.block_size} tokens, kernels {getattr(self.kernels, 'name', '?')}")

    def step(self, entries: Sequence[dict], end: Sequence = ()) -> Optional[torch.Tensor]:
        """Runs one step of the trace; returns float32 logits ``[wanted, vocab]`` or None."""
        batch: List[StepEntry] = []
        for e in entries:
            key = str(e["id"])
            if key not in self.ids:
                self.ids[key] = self._next
                self._next += 1
                self.cache.admit(self.ids[key])
            batch.append(StepEntry(self.ids[key], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = self.runner.run(batch) if batch else None
        for key in end:
            rid = self.ids.pop(str(key), None)
            if rid is not None:
                self.cache.release(rid)
        return logits
