"""A request and its life: WAITING -> PREFILL -> DECODE -> FINISHED (reference: ``serving/request.py:41-86``)."""

from __future__ import annotations

import enum
import itertools
from dataclasses import dataclass, field
from typing import List, Optional

from ..sampling.params import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    PREFILL = "prefill"
    DECODE = "decode"
    FINISHED = "finished"


_ids = itertools.count(1)


@dataclass
class Request:
    prompt_tokens: List[int]
    params: SamplingParams
    id: int = field(default_factory=lambda: next(_ids))
    state: RequestState = RequestState.WAITING
    slot: Optional[int] = None
    num_computed: int = 0            # tokens whose keys and values are in the cache
    cached_prefix_len: int = 0       # prompt tokens taken from pages of an equal prefix
    generated: List[int] = field(default_factory=list)   # the tokens the host has read
    eos_hit: bool = False
    pending: int = 0                 # tokens sampled on the device that the host has not read yet
    pending_row: int = -1            # row of the latest of them among its step's sampled tokens

    @property
    def prompt_len(self) -> int:
        return len(self.prompt_tokens)

    @property
    def num_generated(self) -> int:
        return len(self.generated)

    @property
    def max_new_tokens(self) -> int:
        return self.params.max_new_tokens

    @property
    def context_len(self) -> int:
        return self.prompt_len + self.num_generated + self.pending

    @property
    def last_token(self) -> int:
        return self.generated[-1] if self.generated else self.prompt_tokens[-1]

    def should_finish(self) -> bool:
        return self.eos_hit or self.num_generated >= self.max_new_tokens

    def __repr__(self) -> str:
        return (f"Request(id={self.id}, state={self.state.value}, slot={self.slot}, computed={self.num_computed}, "
                f"prompt={self.prompt_len}, gen={self.num_generated})")
