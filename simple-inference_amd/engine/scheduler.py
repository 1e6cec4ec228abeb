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
from typing import Callable, Deque, List, Optional, Tuple

from .request import Request, RequestState

Gate = Optional[Callable[[Request], bool]]


class Scheduler:
    def __init__(self, max_running: int, token_budget: int, chunk_tokens: int):
        if max_running <= 0 or chunk_tokens <= 0:
            raise ValueError("max_running and chunk_tokens must be positive")
        self.max_running = max_running
        self.token_budget = token_budget
        self.chunk_tokens = chunk_tokens
        self.queue: Deque[Request] = deque()     # not yet let in, oldest first
        self.live: List[Request] = []            # let in and not yet retired, in the order they came in

    def submit(self, req: Request) -> None:
        if req.state is not RequestState.WAITING:
            raise ValueError(f"request {req.id} is {req.state.value}; only a waiting request can be queued")
        self.queue.append(req)

    def busy(self) -> bool:
        return bool(self.queue) or bool(self.live)

    def clear(self) -> None:
        self.queue.clear()
        self.live.clear()

    def retire(self) -> List[Request]:
        """Takes the finished requests out; returns them."""
        gone = [r for r in self.live if r.state is RequestState.FINISHED]
        if gone:
            self.live = [r for r in self.live if r.state is not RequestState.FINISHED]
        return gone

    def let_in(self, gate: Gate = None) -> Optional[Request]:
        """The head of the queue comes in if slot, budget and ``gate`` allow; returns it, or None.  ``gate`` is
        expected to give the request its slot and pages (``Request.enter``); without one it just turns to PREFILL."""
        if not self.queue or len(self.live) >= self.max_running:
            return None
        head = self.queue[0]
        if self.live and sum(r.context_len for r in self.live) + head.prompt_len > self.token_budget:
            return None
        if gate is not None and not gate(head):
            return None
        self.queue.popleft()
        if head.state is RequestState.WAITING:
            head.state = RequestState.PREFILL
        self.live.append(head)
        return head

    def plan(self, gate: Gate = None, admit: bool = True) -> List[Tuple[Request, int]]:
        """(request, number of its next tokens) for one step: decoded tokens first, then prompt portions, then the
        first portions of requests that come in with this step (none with ``admit`` False)."""
        step: List[Tuple[Request, int]] = [(r, 1) for r in self.live if r.state is RequestState.DECODE]
        room = self.chunk_tokens - len(step)
        for r in self.live:
            if room <= 0:
                break
            if r.state is RequestState.PREFILL:
                n = r.tokens_wanted(room)
                step.append((r, n))
                room -= n
        while admit and room > 0:
            newcomer = self.let_in(gate)
            if newcomer is None:
                break
            n = newcomer.tokens_wanted(room)
            step.append((newcomer, n))
            room -= n
        return step

    def __repr__(self) -> str:
        return f"<scheduler: {len(self.queue)} queued, {len(self.live)} of {self.max_running} slots live>"
