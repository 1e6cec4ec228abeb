"""Turns logits rows into tokens with the device sampling kernel."""

from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from .params import SamplingParams, uniforms_for


class _Mirror:
    """A pinned host buffer for four numbers a row (temperature, top-p, uniform number, top-k as int32 bits; a call
    of n rows fills its first 4 n entries, quantity by quantity) and the event of the last copy out of it: the host
    may write into it again once that copy has run."""

    def __init__(self, capacity: int, pinned: bool):
        self.capacity = capacity
        self.pinned = torch.zeros((4 * capacity,), dtype=torch.float32, pin_memory=pinned)
        self.floats = self.pinned.numpy()
        self.ints = self.floats.view(np.int32)
        self.copied = torch.cuda.Event() if pinned else None     # a copy within host memory has run when it returns
        self.in_use = False


class Sampler:
    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = torch.device(device)
        self._mirrors: List[_Mirror] = []     # two, used in turn: a step may be prepared while the last one's copy waits
        self._turn = 0

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], draw_indices: Sequence[int]) -> List[int]:
        """One token per row of float32 ``logits``; row i uses ``params[i]`` and its ``draw_indices[i]``-th draw."""
        tokens = self.sample_on_device(logits, params, draw_indices)
        return tokens.tolist()

    def _mirror_for(self, rows: int) -> _Mirror:
        on_gpu = self.device.type == "cuda"
        if len(self._mirrors) < 2:
            self._mirrors.append(_Mirror(max(64, rows), on_gpu))
            return self._mirrors[-1]
        self._turn ^= 1
        mirror = self._mirrors[self._turn]
        if mirror.in_use and mirror.copied is not None:
            mirror.copied.synchronize()       # long done, unless the host is more than a step ahead
        if mirror.capacity < rows:
            mirror = self._mirrors[self._turn] = _Mirror(max(rows, 2 * mirror.capacity), on_gpu)
        return mirror

    def sample_on_device(self, logits, params, draw_indices) -> torch.Tensor:
        rows = logits.shape[0]
        if rows != len(params) or rows != len(draw_indices):
            raise ValueError(f"{rows} logits rows, {len(params)} parameter sets, {len(draw_indices)} draw indices")
        if all(p.greedy for p in params):    # nothing but the logits is needed: no parameter tensors, no copies
            return self.kernels.sample(logits, None, None, None, None, all_greedy=True)
        # The parameters go over in one copy from pinned memory that the host does not wait for: it is free to
        # prepare the next step while this one's kernels are still queued.
        mirror = self._mirror_for(rows)
        top_k = [p.top_k for p in params]
        top_p = [p.top_p for p in params]
        mirror.floats[0:rows] = [p.temperature for p in params]
        mirror.floats[rows:2 * rows] = top_p
        mirror.floats[2 * rows:3 * rows] = uniforms_for([p.seed for p in params], draw_indices)
        mirror.ints[3 * rows:4 * rows] = top_k
        dev = torch.empty((4, rows), dtype=torch.float32, device=self.device)
        dev.view(-1).copy_(mirror.pinned[:4 * rows], non_blocking=True)
        if mirror.copied is not None:
            mirror.copied.record()
        mirror.in_use = True
        filters = (1 if any(k > 0 for k in top_k) else 0) | (2 if any(0.0 < p < 1.0 for p in top_p) else 0)
        return self.kernels.sample(logits, dev[0], dev[3].view(torch.int32), dev[1], dev[2], filters=filters)
