"""Turns logits rows into tokens with the device sampling kernel."""

from __future__ import annotations

from typing import List, Sequence

import torch

from .params import SamplingParams, uniform_for


class Sampler:
    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], draw_indices: Sequence[int]) -> List[int]:
        """One token per row of float32 ``logits``; row i uses ``params[i]`` and its ``draw_indices[i]``-th draw."""
        tokens = self.sample_on_device(logits, params, draw_indices)
        return tokens.tolist()

    def sample_on_device(self, logits, params, draw_indices) -> torch.Tensor:
        rows = logits.shape[0]
        if rows != len(params) or rows != len(draw_indices):
            raise ValueError(f"{rows} logits rows, {len(params)} parameter sets, {len(draw_indices)} draw indices")
        if all(p.greedy for p in params):    # nothing but the logits is needed: no parameter tensors, no copies
            return self.kernels.sample(logits, None, None, None, None, all_greedy=True)
        host = torch.empty((4, rows), dtype=torch.float32)
        for i, (p, n) in enumerate(zip(params, draw_indices)):
            host[0, i] = p.temperature
            host[1, i] = p.top_p
            host[2, i] = 0.0 if p.greedy else uniform_for(p.seed, n)
        top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32)
        dev = host.to(self.device)
        filters = (1 if any(p.top_k > 0 for p in params) else 0) | (2 if any(0.0 < p.top_p < 1.0 for p in params) else 0)
        return self.kernels.sample(logits, dev[0], top_k.to(self.device), dev[1], dev[2], filters=filters)
