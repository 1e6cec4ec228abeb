"""A request: what was asked, and the books of how far it has come.

Its life is WAITING -> PREFILL -> DECODE -> FINISHED, as in the reference (``serving/request.py:41-86``).
The request keeps its own books and makes its own transitions: the scheduler asks it how many tokens
it would bring to a step (``tokens_wanted``), the engine asks for those tokens (``take``), tells it that
a token was sampled for it on the device (``sampled``) and later hands it the token (``deliver``).
Between ``sampled`` and ``deliver`` the token is *in flight*: it counts towards the request's length,
so that plans and admission see the same numbers whether or not the engine runs a step ahead.
"""

from __future__ import annotations

import enum
import itertools
from typing import List, Optional, Sequence, Tuple

from ..sampling.params import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    PREFILL = "prefill"
    DECODE = "decode"
    ENDING = "ending"        # its last token is sampled but not read yet; pages and slot are given back already
    FINISHED = "finished"


_next_id = itertools.count(1)


class Request:
    __slots__ = ("id", "prompt_tokens", "params", "state", "slot", "num_computed", "cached_prefix_len", "generated",
                 "finish_reason", "in_flight", "in_flight_row")

    def __init__(self, prompt_tokens: Sequence[int], params: SamplingParams, id: Optional[int] = None):
        self.id = next(_next_id) if id is None else id
        self.prompt_tokens: List[int] = list(prompt_tokens)
        self.params = params
        self.state = RequestState.WAITING
        self.slot: Optional[int] = None
        self.num_computed = 0            # tokens whose keys and values are in the cache
        self.cached_prefix_len = 0       # of those, prompt tokens found in pages of an equal prefix
        self.generated: List[int] = []   # the tokens the host has read
        self.finish_reason: Optional[str] = None    # "eos" or "length" once FINISHED
        self.in_flight = 0               # tokens sampled on the device that the host has not read yet
        self.in_flight_row = -1          # row of the latest of them among its step's sampled tokens

    # -- what the books say --------------------------------------------------------------
    prompt_len = property(lambda self: len(self.prompt_tokens))
    num_generated = property(lambda self: len(self.generated))
    max_new_tokens = property(lambda self: self.params.max_new_tokens)
    eos_hit = property(lambda self: self.finish_reason == "eos")

    @property
    def context_len(self) -> int:
        return len(self.prompt_tokens) + len(self.generated) + self.in_flight

    @property
    def total_len(self) -> int:
        """The most positions the request can ever hold: what admission has to find pages for."""
        return len(self.prompt_tokens) + self.params.max_new_tokens

    def tokens_wanted(self, room: int) -> int:
        """How many tokens it would bring to a step that has ``room`` left."""
        if self.state is RequestState.DECODE:
            return 1
        if self.state is RequestState.PREFILL:
            return max(0, min(room, len(self.prompt_tokens) - self.num_computed))
        return 0

    def length_is_certain_after_next_token(self) -> bool:
        """False if the token it is about to get may be its last by count (an end-of-sequence token is only
        known once the token has been read)."""
        return len(self.generated) + self.in_flight < self.params.max_new_tokens

    def last_token_is_in_flight(self) -> bool:
        """True if the token that has been sampled for it and not read yet is its last by count, whatever it is."""
        return (self.state is RequestState.DECODE and self.in_flight > 0
                and len(self.generated) + self.in_flight >= self.params.max_new_tokens)

    # -- transitions ---------------------------------------------------------------------
    def enter(self, slot: int, reused_tokens: int = 0) -> None:
        """Admitted: it has a slot, and ``reused_tokens`` of its prompt are in the cache already."""
        self.slot = slot
        self.cached_prefix_len = self.num_computed = reused_tokens
        self.state = RequestState.PREFILL

    def take(self, n: int) -> Tuple[List[int], bool, Optional[int]]:
        """Its next ``n`` tokens for a step: (token ids, whether the last of them gets a token sampled, the row of
        the device's sampled tokens that holds its one token if the host has not read it yet).  Books them as run."""
        if self.state is RequestState.DECODE:
            if n != 1:
                raise ValueError(f"request {self.id} decodes one token a step, not {n}")
            self.num_computed += 1
            if self.in_flight:
                return [0], True, self.in_flight_row
            return [self.generated[-1] if self.generated else self.prompt_tokens[-1]], True, None
        if self.state is not RequestState.PREFILL or not 0 < n <= len(self.prompt_tokens) - self.num_computed:
            raise ValueError(f"request {self.id} ({self.state.value}) cannot bring {n} tokens")
        tokens = self.prompt_tokens[self.num_computed:self.num_computed + n]
        self.num_computed += n
        return tokens, self.num_computed == len(self.prompt_tokens), None

    def sampled(self, row: int) -> None:
        """A token was sampled for it, row ``row`` of its step's tokens; a prompt that has just ended decodes from
        the next step on."""
        self.state = RequestState.DECODE
        self.in_flight += 1
        self.in_flight_row = row

    def end_ahead(self) -> None:
        """Its last token is in flight: it takes part in no later step and holds nothing any more; ``deliver`` ends
        it when the token is read."""
        if not self.last_token_is_in_flight():
            raise ValueError(f"request {self.id} cannot end before its tokens are read: {self!r}")
        self.state = RequestState.ENDING
        self.slot = None

    def deliver(self, token: int, eos_ids=()) -> bool:
        """The host has read a sampled token.  False if the request had ended before (the token was sampled a step
        too far and is dropped); otherwise the token is booked, and the request ends if it was an end-of-sequence
        token (kept in ``generated``; reference: ``serving/engine.py:449-460``) or the last one allowed."""
        self.in_flight -= 1
        if self.state is RequestState.FINISHED:
            return False
        self.generated.append(token)
        if token in eos_ids and not self.params.ignore_eos:
            self.finish_reason = "eos"
        elif len(self.generated) >= self.params.max_new_tokens:
            self.finish_reason = "length"
        if self.finish_reason is not None:
            self.state = RequestState.FINISHED
            self.slot = None
        return True

    def __repr__(self) -> str:
        return (f"<request {self.id} {self.state.value}: {self.num_computed}/{len(self.prompt_tokens)} prompt tokens run, "
                f"{len(self.generated)} generated, {self.in_flight} in flight>")
