"""The scheduler: who runs in the next step, with how many tokens, and who may come in.

One decision a step, ``plan``: every decoding request gets its one token, then the requests that are
still on their prompts get portions, in the order they came in, until ``chunk_tokens`` tokens are in
the step; into whatever room is left, requests are let in from the head of the queue and get their
first portion at once.  So a request enters only in a step that can run some of its tokens: it does
not hold a promise of pages while it could not run anyway, and prompts that arrive together are
matched against the prefix cache after the earlier ones have written their pages.

The rules of coming in are the reference's (``serving/scheduler.py:93-123``): first come first served;
a free slot; the context already inside plus the newcomer's prompt within ``token_budget`` (an empty
engine takes any one request); and the caller's ``gate`` (the cache manager promising its pages).  If
the head of the queue cannot come in, nobody behind it does.  Nothing is ever put out again: a request
is promised the pages of its whole declared length before it starts, so pages cannot run out in
mid-flight; when the pool is full the head of the queue waits until a finished request gives its
pages back.  The cut of prompts into portions has no counterpart in the reference (``plan.md:811-868``
sketches it).
"""

from __future__ import annotations

from collections import deque
from typing import Callable, Deque, Iterator, List, Optional, Tuple

from .request import Request, RequestState

Gate = Optional[Callable[[Request], bool]]
Share = Tuple[Request, int]      # a request and the number of its next tokens that a step runs


class Scheduler:
    def __init__(self, max_running: int, token_budget: int, chunk_tokens: int):
        for name, value in (("max_running", max_running), ("chunk_tokens", chunk_tokens)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        self.max_running, self.token_budget, self.chunk_tokens = max_running, token_budget, chunk_tokens
        self.queue: Deque[Request] = deque()     # not yet let in, oldest first
        self.live: List[Request] = []            # let in and not yet retired, in the order they came in

    # -- one step ------------------------------------------------------------------------
    def plan(self, gate: Gate = None, admit: bool = True) -> List[Share]:
        """The shares of one step: decoded tokens first, then prompt portions, then the first portions of requests
        that come in with this step (none with ``admit`` False)."""
        room = self.chunk_tokens
        shares: List[Share] = []
        for req in self._in_state(RequestState.DECODE):
            shares.append((req, 1))
            room -= 1
        sources = [self._in_state(RequestState.PREFILL)]
        if admit:
            sources.append(self._newcomers(gate))
        for source in sources:
            while room > 0:     # asked before the next request is: nobody comes in for nothing
                req = next(source, None)
                if req is None:
                    break
                n = req.tokens_wanted(room)
                shares.append((req, n))
                room -= n
        return shares

    def _in_state(self, state: RequestState) -> Iterator[Request]:
        return (req for req in self.live if req.state is state)

    def _newcomers(self, gate: Gate) -> Iterator[Request]:
        """Requests as they come in, for as long as the head of the queue may (asked for one at a time: nobody comes
        in whom the step has no room for)."""
        while True:
            req = self.let_in(gate)
            if req is None:
                return
            yield req

    # -- coming and going ------------------------------------------------------------------
    def let_in(self, gate: Gate = None) -> Optional[Request]:
        """The head of the queue comes in if slot, budget and ``gate`` allow; returns it, or None.  ``gate`` is
        expected to give the request its slot and pages (``Request.enter``); without one it just turns to PREFILL."""
        head = self.queue[0] if self.queue else None
        if head is None or not self._has_room_for(head) or not (gate is None or gate(head)):
            return None
        self.live.append(self.queue.popleft())
        if head.state is RequestState.WAITING:
            head.state = RequestState.PREFILL
        return head

    def _has_room_for(self, newcomer: Request) -> bool:
        if len(self.live) >= self.max_running:
            return False
        if not self.live:
            return True             # an empty engine takes any one request, however long
        inside = 0
        for req in self.live:
            inside += req.context_len
        return inside + newcomer.prompt_len <= self.token_budget

    def retire(self) -> List[Request]:
        """Takes out the requests that have finished, or will with a token that is sampled already; returns them."""
        staying: List[Request] = []
        gone: List[Request] = []
        for req in self.live:
            (gone if req.state in (RequestState.FINISHED, RequestState.ENDING) else staying).append(req)
        if gone:
            self.live = staying
        return gone

    def submit(self, req: Request) -> None:
        if req.state is not RequestState.WAITING:
            raise ValueError(f"request {req.id} is {req.state.value}; only a waiting request can be queued")
        self.queue.append(req)

    def busy(self) -> bool:
        return len(self.queue) + len(self.live) > 0

    def clear(self) -> None:
        self.queue.clear()
        del self.live[:]

    def __repr__(self) -> str:
        return f"<scheduler: {len(self.queue)} queued, {len(self.live)} of {self.max_running} slots live>"
