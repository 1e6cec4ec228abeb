"""What parts are built with and what a step hands to them."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional

import torch


@dataclass
class BuildEnv:
    """Where and with what a model's parts are built."""

    kernels: Any            # the object that launches the device kernels
    device: torch.device
    dtype: torch.dtype      # compute dtype: torch.bfloat16 or torch.float32
    max_positions: int      # absolute positions the engine will ever use (sizes rotation tables)
    _shared: Dict[Any, Any] = field(default_factory=dict)  # parts shared between layers, by spec key


@dataclass
class StepContext:
    """One batch of tokens: runs of consecutive tokens of several requests.

    Token ``t`` of the flat batch belongs to sequence ``seq_of_token[t]`` and stands
    at absolute position ``positions[t]``.  Sequence ``s`` brings tokens
    ``cu_q[s] .. cu_q[s+1]`` and holds ``kv_len[s]`` tokens once the step is done,
    so its first new token stands at ``kv_len[s] - (cu_q[s+1] - cu_q[s])``.
    All tensors are int32 on the device.
    """

    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    seq_of_token: torch.Tensor
    cu_q: torch.Tensor
    kv_len: torch.Tensor
    state_slots: torch.Tensor
    logit_rows: Optional[torch.Tensor]
    n_logit_rows: int
    max_q_len: int          # host-side facts for choosing kernels and grids
    max_kv_len: int
    kernels: Any = None
    block_tables: list = field(default_factory=list)  # one [n_seqs, width] table per cache group
    n_decode_seqs: int = 0  # sequences 0 .. n_decode_seqs-1 bring exactly one token (they are sorted first)
    q_lens: list = field(default_factory=list)  # host copy: tokens each sequence brings
    kv_bound: int = 0  # replayed graphs: an upper bound of kv_len that fixes grids (0: use max_kv_len)
    max_run_kv_len: int = 0  # the longest kv_len among the sequences that bring more than one token (0: not known)
    extra: dict = field(default_factory=dict)  # name -> int32 [n_tokens]: what the step's entries brought beside tokens


@dataclass
class LayerCache:
    """What one run of one layer may touch of the caches in this step."""

    k_pages: Optional[torch.Tensor] = None      # [pages, kv_heads, page_size, head_dim]
    v_pages: Optional[torch.Tensor] = None      # [pages, kv_heads, head_dim, page_size]
    block_table: Optional[torch.Tensor] = None  # [n_seqs, max_pages] int32, -1 where no page
    page_size: int = 0
    state: Optional[torch.Tensor] = None        # [slots, *state_shape]; row = ctx.state_slots[s]


class ResidualStream:
    """The hidden state between parts: a 32-bit residual and a delta not yet added.

    Parts produce deltas in the compute dtype; the sum over the residual is kept
    in float32 in both modes.  The add is fused into the norm that follows it.

    A part may leave its last product uncomputed (an object with ``compute()``, as the kernels'
    ``pending_linear`` returns): ``raw_delta`` shows it to a norm that can have it computed
    straight into the residual; ``delta`` computes it for everybody else.
    """

    __slots__ = ("residual", "raw_delta")

    def __init__(self, residual: torch.Tensor, delta: Optional[torch.Tensor] = None):
        self.residual = residual
        self.raw_delta = delta

    @property
    def delta(self):
        if hasattr(self.raw_delta, "compute"):
            self.raw_delta = self.raw_delta.compute()
        return self.raw_delta

    @delta.setter
    def delta(self, value):
        self.raw_delta = value
