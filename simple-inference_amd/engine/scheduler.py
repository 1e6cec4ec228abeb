"""The scheduler: who is admitted, and which tokens of whom a step runs.

Admission is the reference's (``serving/scheduler.py:93-123``): first come first served; while
there is a waiting request and a free slot, the head of the queue is admitted if the context
already admitted plus its prompt fits ``token_budget`` (an idle engine always admits one) and if
``can_admit`` (the cache manager promising its pages) says yes.  If the head cannot be admitted
nobody behind it is: no overtaking.  Nothing is ever preempted: a request is promised the pages
of its whole declared length before it starts, so pages cannot run out in mid-flight; when the
pool is full the head of the queue waits until a finished request gives its pages back.

What the reference lacks is the cut of prompts into portions (``plan.md:811-868`` sketches it).
``plan_step`` gives every decoding request its one token first, then hands prompt portions to
the prefilling requests in admission order until ``chunk_tokens`` tokens are in the step.  A
request turns to DECODE in the step that runs its last prompt token and emits its first token
from that step.

Given the admission test, ``plan_step`` also admits: a waiting request enters only in a step
that still has room for its first prompt tokens.  So a request is not promised pages while it
could not run anyway, and when prompts arrive together the later ones are matched against the
prefix cache after the earlier ones have written their pages, not before.
"""

from __future__ import annotations

from collections import deque
from typing import Callable, Deque, List, Optional, Tuple

from .request import Request, RequestState


class Scheduler:
    def __init__(self, max_running: int, token_budget: int, chunk_tokens: int):
        if max_running <= 0 or chunk_tokens <= 0:
            raise ValueError("max_running and chunk_tokens must be positive")
        self.max_running = max_running
        self.token_budget = token_budget
        self.chunk_tokens = chunk_tokens
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []

    def add(self, req: Request) -> None:
        req.state = RequestState.WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def evict_finished(self) -> List[Request]:
        done = [r for r in self.running if r.state is RequestState.FINISHED]
        if done:
            self.running = [r for r in self.running if r.state is not RequestState.FINISHED]
        return done

    def _running_tokens(self) -> int:
        return sum(r.context_len for r in self.running)

    def admit(self, can_admit: Optional[Callable[[Request], bool]] = None,
              limit: Optional[int] = None) -> List[Request]:
        """Admits from the head of the queue while slots, the token budget and ``can_admit`` allow, at most
        ``limit`` requests."""
        admitted: List[Request] = []
        used = self._running_tokens()
        while self.waiting and len(self.running) < self.max_running and (limit is None or len(admitted) < limit):
            head = self.waiting[0]
            if (self.running or admitted) and used + head.prompt_len > self.token_budget:
                break
            if can_admit is not None and not can_admit(head):
                break
            self.waiting.popleft()
            head.state = RequestState.PREFILL
            self.running.append(head)
            admitted.append(head)
            used += head.prompt_len
        return admitted

    def plan_step(self, can_admit: Optional[Callable[[Request], bool]] = None,
                  admit: bool = False) -> List[Tuple[Request, int]]:
        """(request, number of its next tokens) for one step: decoded tokens, then prompt portions.

        With ``admit`` (or an admission test), waiting requests are admitted one by one while the step
        has room left for prompt tokens, and get their first portion in this step."""
        plan: List[Tuple[Request, int]] = []
        room = self.chunk_tokens
        for r in self.running:
            if r.state is RequestState.DECODE:
                plan.append((r, 1))
                room -= 1
        for r in self.running:
            if r.state is RequestState.PREFILL:
                if room <= 0:
                    break
                n = min(room, r.prompt_len - r.num_computed)
                plan.append((r, n))
                room -= n
        if admit or can_admit is not None:
            while room > 0:
                newcomers = self.admit(can_admit, limit=1)
                if not newcomers:
                    break
                r = newcomers[0]
                n = min(room, r.prompt_len - r.num_computed)
                plan.append((r, n))
                room -= n
        return plan

    def __repr__(self) -> str:
        return f"Scheduler(waiting={len(self.waiting)}, running={len(self.running)}/{self.max_running})"
