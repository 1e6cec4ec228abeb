"""The engine: requests in, tokens out (reference: ``serving/engine.py:95-517``).

``add_request`` queues a request; ``step`` runs one iteration: finished requests leave, the
scheduler picks this step's tokens (one per decoding request, then prompt portions) and admits
waiting requests into the room that is left while slots, token budget and pages allow, ONE call
of the step function runs them all as one batch, and the sampler turns the returned logits into
tokens.  ``run`` steps
until nothing is left.  The reference's step runs two forwards instead, one for whole prompts
and one for decoded tokens (``serving/engine.py:330-349``).

Running ahead: a decoding request's next input token is the sampler's output of the step before, which is on
the device.  Who takes part in the next step, and with how many tokens, depends on the sampled tokens only through
the ends of requests.  So the next step is always planned and launched (admission included) before the host waits
for the tokens of the step on the GPU, its token ids copied on the device; the GPU works while the host reads,
books and plans.  The one end the host knows without reading a token is the end by count: a request whose token
in flight is its last ends ahead (``ENDING``), takes part in no later step, and gives its pages and slot back
before the next step is planned.  ``step`` still reports one step's tokens per call, in order.  A request that
turns out to have ended on an end-of-sequence token has then run one token too far; that token is dropped, and its
slot goes to the next request a step later.
"""

from __future__ import annotations

import sys
import time
from typing import Dict, Iterator, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .build import default_kernels, model_from_folder, model_from_random
from .ranges import NamedRanges
from .request import Request, RequestState
from .scheduler import Scheduler
from .graphs import GraphedDecode, GraphUnavailable
from .step import StepEntry, StepRunner


class Engine:
    def __init__(self, model, model_cfg, engine_cfg: EngineConfig, kernels):
        self.model = model
        self.model_cfg = model_cfg
        self.cfg = engine_cfg
        self.kernels = kernels
        self.device = torch.device(engine_cfg.device)
        self.max_seq_len = engine_cfg.max_seq_len
        plan = model.plan
        if engine_cfg.eos_id is None:
            self.eos_ids = tuple(plan.eos_token_ids)
        elif engine_cfg.eos_id < 0:
            self.eos_ids = ()
        else:
            self.eos_ids = (engine_cfg.eos_id,)
        self.cache = CacheManager(
            model.cache_layout(), page_size=engine_cfg.block_size, num_pages=engine_cfg.resolved_num_kv_blocks(),
            max_running=engine_cfg.max_running, dtype=engine_cfg.torch_dtype, device=self.device)
        self.runner = StepRunner(model, self.cache, kernels, self.device, engine_cfg.max_seq_len)
        self.scheduler = Scheduler(engine_cfg.max_running, engine_cfg.resolved_token_budget(),
                                   engine_cfg.chunk_tokens)
        self.sampler = Sampler(kernels, self.device)
        self.prefix_cache = None
        if engine_cfg.use_prefix_cache:
            from ..cache.prefix import PrefixCache
            cap = engine_cfg.prefix_cache_blocks or engine_cfg.resolved_num_kv_blocks()
            self.prefix_cache = PrefixCache(self.cache, max_pages=cap)
        self.graphs = None
        if engine_cfg.graphs_wanted():
            self.graphs = GraphedDecode(self)
        self.stats = {"steps": 0, "tokens_run": 0, "prefill_tokens": 0, "decode_tokens": 0, "steps_ahead": 0,
                      "graph_fallbacks": 0}
        self.ranges = NamedRanges(engine_cfg.profile_ranges)
        self._ahead = None   # a step launched but not yet read: (requests that sampled a token, those tokens)
        self._token_mirrors = None   # two pinned host buffers that sampled tokens are copied into, in turn
        self._mirror_turn = 0
        self.model_folder = None   # where the model came from, if from a folder: a tokenizer file may lie beside it
        self._tokenizer = None
        if engine_cfg.warmup:
            self.warmup()

    # -- construction ----------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, engine_cfg: Optional[EngineConfig] = None, kernels=None) -> "Engine":
        engine_cfg = engine_cfg or EngineConfig()
        kernels = kernels if kernels is not None else default_kernels()
        model, model_cfg = model_from_folder(folder, engine_cfg, kernels)
        engine = cls(model, model_cfg, engine_cfg, kernels)
        engine.model_folder = folder
        return engine

    @classmethod
    def from_random(cls, config_dict, seed: int = 0, engine_cfg: Optional[EngineConfig] = None, kernels=None,
                    **random_options) -> "Engine":
        engine_cfg = engine_cfg or EngineConfig()
        kernels = kernels if kernels is not None else default_kernels()
        model, model_cfg = model_from_random(config_dict, seed, engine_cfg, kernels, **random_options)
        return cls(model, model_cfg, engine_cfg, kernels)

    def describe(self) -> str:
        """One line about the loaded model: parameters and cache bytes a token."""
        from .build import describe
        return describe(self.model, self.model_cfg, self.cfg)

    # -- requests ----------------------------------------------------------------
    def add_request(self, prompt_tokens: Sequence[int], max_new_tokens: Optional[int] = None,
                    params: Optional[SamplingParams] = None) -> Request:
        """Queues a request (reference: ``serving/engine.py:228-254``, same checks)."""
        prompt = [int(t) for t in prompt_tokens]
        if params is None:
            params = SamplingParams(max_new_tokens=max_new_tokens if max_new_tokens is not None else 16)
        elif max_new_tokens is not None:
            params = SamplingParams(**{**params.__dict__, "max_new_tokens": max_new_tokens})
        if not prompt:
            raise ValueError("prompt_tokens is empty")
        total = len(prompt) + params.max_new_tokens
        if total > self.max_seq_len:
            raise ValueError(f"prompt_len ({len(prompt)}) + max_new_tokens ({params.max_new_tokens}) "
                             f"> max_seq_len ({self.max_seq_len})")
        for g in self.cache.groups:
            need = g.pages_to_reserve(total, self.cfg.chunk_tokens)
            if need > g.num_pages:
                raise ValueError(f"request needs more pages than the whole cache: {need} > {g.num_pages}")
        vocab = self.model.vocab_size
        if any(t < 0 or t >= vocab for t in prompt):
            raise ValueError("prompt contains out-of-range token ids")
        req = Request(prompt, params)
        self.scheduler.submit(req)
        return req

    def has_work(self) -> bool:
        return self.scheduler.busy() or self._ahead is not None

    def reset(self) -> None:
        """Drops every request and gives every page and slot back."""
        self.scheduler.clear()
        self._ahead = None
        self.cache.reset()
        if self.prefix_cache is not None:
            self.prefix_cache.clear()

    # -- admission ----------------------------------------------------------------
    def _try_admit(self, req: Request) -> bool:
        """The scheduler's gate: finds the request a slot and the pages of its whole length (those of an equal
        prefix by reference) and lets it enter, or says no."""
        shared: List[int] = []
        if self.prefix_cache is not None:
            shared = self.prefix_cache.match(req.prompt_tokens)
            if self._prefix_still_being_written(req, len(shared)):
                return False
            need = self.cache.groups[0].pages_to_reserve(req.total_len, self.cfg.chunk_tokens) - len(shared)
            if not self.prefix_cache.evict_until_available(need, protected=shared):
                return False
        if not self.cache.can_admit(req.total_len, self.cfg.chunk_tokens, len(shared)):
            return False
        slot = self.cache.admit(req.id, req.total_len, self.cfg.chunk_tokens, shared_pages=shared)
        req.enter(slot, reused_tokens=len(shared) * self.cfg.block_size)
        return True

    def _prefix_still_being_written(self, req: Request, matched_pages: int) -> bool:
        """True if a request that is still running its prompt shares more whole pages with ``req`` than the
        prefix cache holds yet: ``req`` then waits the few steps until they are written, instead of
        computing them a second time."""
        ps = self.cfg.block_size
        reusable = (req.prompt_len - 1) // ps
        if matched_pages >= reusable:
            return False
        for other in self.scheduler.live:
            if other.state is not RequestState.PREFILL:
                continue
            limit = min(reusable, other.prompt_len // ps)
            pages = matched_pages
            while pages < limit and req.prompt_tokens[pages * ps:(pages + 1) * ps] == \
                    other.prompt_tokens[pages * ps:(pages + 1) * ps]:
                pages += 1
            if pages > matched_pages and req.prompt_tokens[:matched_pages * ps] == other.prompt_tokens[:matched_pages * ps]:
                return True
        return False

    # -- one iteration ---------------------------------------------------------------
    @torch.no_grad()
    def step(self) -> Dict[int, int]:
        """Runs one iteration; returns {request id: token} for every request that emitted one."""
        launched = self._ahead
        self._ahead = None
        if launched is None:
            launched = self._launch(None)
            if launched is None:
                return {}
        if self.cfg.run_ahead and launched[0]:
            # The next step is planned before the host waits for this one's tokens.  What it needs to know of them it
            # knows already: a request whose token in flight is its last by count ends now, as far as planning goes
            # (its pages and slot go back: the next step follows this one on the stream, so whoever gets them
            # writes them after this step has read them).  An end-of-sequence token is found out a step late.
            for req in launched[0]:
                if req.last_token_is_in_flight():
                    req.end_ahead()
                    self.cache.release(req.id)
            self._ahead = self._launch(launched)
        return self._collect(*launched)

    def _launch(self, before):
        """Plans a step and puts it on the GPU.  ``before``: the step launched before it whose tokens the host has
        not read (its decoding requests take their input from its sampled tokens on the device), or None.
        Returns (requests that sample a token, their tokens), or None if there is nothing to run."""
        with self.ranges("engine.schedule"):
            self.scheduler.retire()      # their pages and slots went back when they finished
            plan = self.scheduler.plan(self._try_admit)   # lets requests in, too: into steps with room for their tokens
        if not plan:
            return None
        entries, emitters = [], []
        for req, n in plan:
            kind = "decode_tokens" if req.state is RequestState.DECODE else "prefill_tokens"
            tokens, samples, device_row = req.take(n)
            entries.append(StepEntry(req.id, tokens, [n - 1] if samples else [], token_from=device_row))
            if samples:
                emitters.append(req)
            self.stats[kind] += n
            self.stats["tokens_run"] += n
        self.stats["steps"] += 1
        self.stats["steps_ahead"] += before is not None

        device_tokens = before[1][0] if before is not None and before[1] is not None else None
        with self.ranges("engine.forward"):
            logits = self._forward(entries, device_tokens)
        if self.prefix_cache is not None:
            for req, _ in plan:
                if req.state is RequestState.PREFILL:
                    # pages a prompt has filled so far can be shared from the next step on
                    self.prefix_cache.insert(req.prompt_tokens[:req.num_computed], self.cache.table(0, req.id))
        if not emitters:
            return [], None
        with self.ranges("engine.sample"):
            tokens = self._sample(logits, emitters, [r.num_generated + r.in_flight for r in emitters])
        for row, req in enumerate(emitters):
            req.sampled(row)
        return emitters, tokens

    def _forward(self, entries: List[StepEntry], device_tokens):
        """One call of the step function: a replayed graph where the step is one token for every request, else
        eager.  A graph that cannot be captured or replayed is given up for good (reference:
        ``serving/engine.py:300-309,478-497``): the same entries run eagerly, on the books as they were."""
        if self.graphs is not None and self.graphs.can_run(entries):
            try:
                return self.graphs.run(entries, device_tokens)
            except GraphUnavailable as exc:
                self._give_up_graphs(exc)
        return self.runner.run(entries, device_tokens)

    def _give_up_graphs(self, exc) -> None:
        cause = exc.__cause__ or exc
        print(f"[engine] graph replay failed ({type(cause).__name__}: {cause}); decode steps run eagerly from here on",
              file=sys.stderr, flush=True)
        self.graphs = None
        self.stats["graph_fallbacks"] += 1

    def _sample(self, logits, emitters: List[Request], draw_indices: List[int]):
        """Samples on the device and starts the copy of the tokens to the host right behind the sampler, so that
        work launched later does not stand between the tokens and the host.  Returns (device tokens, read) where
        ``read()`` waits for the copy and gives the tokens as a list."""
        tokens = self.sampler.sample_on_device(logits, [r.params for r in emitters], draw_indices)
        if self.device.type != "cuda":
            return tokens, tokens.tolist
        if self._token_mirrors is None:
            rows = max(self.cfg.max_running, self.cfg.chunk_tokens)
            self._token_mirrors = [(torch.empty(rows, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                                   for _ in range(2)]
        self._mirror_turn ^= 1
        mirror, copied = self._token_mirrors[self._mirror_turn]
        n = tokens.numel()
        mirror[:n].copy_(tokens, non_blocking=True)
        copied.record()

        def read():
            copied.synchronize()
            return mirror[:n].tolist()
        return tokens, read

    def _collect(self, emitters: List[Request], tokens) -> Dict[int, int]:
        """Reads a launched step's sampled tokens and books them.  A request that ends gives its pages and slot
        back at once: the next step may hand them out.  One that had ended on an end-of-sequence token a step ago
        (this step ran ahead of that news) drops its token."""
        emitted: Dict[int, int] = {}
        if not emitters:
            return emitted
        with self.ranges("engine.collect"):
            for req, token in zip(emitters, tokens[1]()):
                if req.deliver(int(token), self.eos_ids):
                    emitted[req.id] = int(token)
                    if req.state is RequestState.FINISHED and req.id in self.cache.lengths:
                        self.cache.release(req.id)      # unless it went back when the request ended ahead
        return emitted

    def run(self) -> Dict[int, Request]:
        """Steps until every queued request has finished; returns them by id."""
        seen: Dict[int, Request] = {r.id: r for r in (*self.scheduler.queue, *self.scheduler.live)}
        while self.has_work():
            self.step()
            seen.update((r.id, r) for r in self.scheduler.live)
        return seen

    def warmup(self, num_seqs: int = 2, prompt_len: int = 8, decode_steps: int = 4) -> None:
        """Runs dummy requests through prefill and decode, then resets (reference: ``serving/engine.py:277-312``)."""
        num_seqs = max(1, min(num_seqs, self.cfg.max_running))
        prompt_len = max(1, min(prompt_len, self.max_seq_len - decode_steps - 1))
        vocab = self.model.vocab_size
        dummy = [i % vocab for i in range(prompt_len)]
        for _ in range(num_seqs):
            self.add_request(dummy, params=SamplingParams(max_new_tokens=decode_steps + 1, ignore_eos=True))
        guard = prompt_len + decode_steps + num_seqs + 8
        while self.has_work() and guard > 0:
            self.step()
            guard -= 1
        if self.graphs is not None:
            try:
                self.graphs.capture_all()
            except GraphUnavailable as exc:
                self._give_up_graphs(exc)
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        self.reset()

    # -- single-stream entry points ------------------------------------------------------
    def tokenizer(self):
        """The text front-end of the model folder (its ``tokenizer.json``); raises where there is none."""
        if self._tokenizer is None:
            if self.model_folder is None:
                raise ValueError("this engine was not built from a model folder, so it has no tokenizer: give token ids")
            from ..tokenizer import Tokenizer
            self._tokenizer = Tokenizer.from_folder(self.model_folder, self.model.plan.bos_token_id)
        return self._tokenizer

    def generate(self, prompt, max_new_tokens: int = 256, temperature: float = 1.0,
                 top_k: int = 50, top_p: float = 0.9, seed: int = 0) -> Iterator:
        """Yields the tokens of one request as they come; stops at EOS without yielding it
        (reference: ``generate.py:50-119``, same option names and defaults).  ``prompt`` is a list of token ids, and
        token ids are yielded; or a text, as the reference takes it, if the model folder holds a ``tokenizer.json``:
        then the pieces of text are yielded that each new token adds to the decoded output."""
        if isinstance(prompt, str):
            tok = self.tokenizer()
            ids, shown = [], ""
            for token in self.generate(tok.encode(prompt, add_bos=True), max_new_tokens, temperature, top_k, top_p,
                                       seed):
                ids.append(token)
                text = tok.decode(ids)
                if text.endswith("\ufffd"):     # half of a character that the next token completes
                    continue
                yield text[len(shown):]
                shown = text
            return
        prompt_tokens = prompt
        req = self.add_request(prompt_tokens, params=SamplingParams(
            temperature=temperature, top_k=top_k, top_p=top_p, seed=seed, max_new_tokens=max_new_tokens))
        sent = 0
        while req.state is not RequestState.FINISHED:
            self.step()
            while sent < len(req.generated):
                token = req.generated[sent]
                sent += 1
                if req.eos_hit and sent == len(req.generated):
                    return
                yield token

    def generate_with_stats(self, prompt_tokens: Sequence[int], max_new_tokens: int = 256, temperature: float = 1.0,
                            top_k: int = 50, top_p: float = 0.9, seed: int = 0, on_token=None):
        """(tokens, stats) with the reference's stat names (``generate.py:227-237``); for a text prompt
        (text, stats), as there."""
        if isinstance(prompt_tokens, str):
            tok = self.tokenizer()
            tokens, stats = self.generate_with_stats(tok.encode(prompt_tokens, add_bos=True), max_new_tokens,
                                                     temperature, top_k, top_p, seed, on_token)
            return tok.decode(tokens), stats
        sync = (lambda: torch.cuda.synchronize(self.device)) if self.device.type == "cuda" else (lambda: None)
        if self.device.type == "cuda":
            torch.cuda.reset_peak_memory_stats(self.device)
        sync()
        t0 = time.perf_counter()
        t_first = None
        out: List[int] = []
        for token in self.generate(prompt_tokens, max_new_tokens, temperature, top_k, top_p, seed):
            if t_first is None:
                sync()
                t_first = time.perf_counter()
            out.append(token)
            if on_token is not None:
                on_token(token)
        sync()
        t1 = time.perf_counter()
        t_first = t_first if t_first is not None else t1
        n = len(out)
        decode_s = t1 - t_first
        stats = {
            "prompt_tokens": len(prompt_tokens), "new_tokens": n,
            "ttft_ms": (t_first - t0) * 1e3, "prefill_ms": (t_first - t0) * 1e3,
            "tpot_ms": decode_s * 1e3 / max(n - 1, 1),
            "decode_tok_s": (n - 1) / decode_s if n > 1 and decode_s > 0 else 0.0,
            "total_wall_ms": (t1 - t0) * 1e3, "total_tok_s": n / (t1 - t0) if t1 > t0 else 0.0,
            "peak_vram_gb": torch.cuda.max_memory_allocated(self.device) / 1e9 if self.device.type == "cuda" else 0.0,
        }
        return out, stats
