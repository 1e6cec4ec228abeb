"""Decode-only steps replayed from captured hipGraphs.

A decode step launches some nine kernels a layer; at small batches the time to launch them
exceeds the time they run.  As the reference does with CUDA graphs (``model/cuda_graph.py:62-88``,
``serving/paged_decoder.py:93-106,260-274``), the whole forward pass of a step in which every
request brings one token is captured once per batch-size bucket (1, 2, 4, ... up to
``max_running``) and replayed afterwards.  The rules are the reference's:

* everything a kernel reads that changes from step to step (token ids, positions, lengths, block
  tables, slots) lives in device buffers of fixed address, filled before each replay; loop bounds
  come from those buffers, grids from the bucket and the engine's ``max_seq_len``;
* pages are taken on the host before the replay (``serving/paged_kv_cache.py:258-270``);
* rows that pad a batch up to its bucket hold token 0 at position 0 and write to the scratch page
  and scratch slot, which no request owns (``serving/paged_decoder.py:224-247``).

``torch.cuda.CUDAGraph`` is hipGraph on this platform; this package's kernels are launched on
torch's current stream, so they are captured with the library products between them.
"""

from __future__ import annotations

import contextlib
import gc
from typing import Dict, List

import numpy as np
import torch

from ..parts.context import StepContext
from .step import StepEntry


class GraphUnavailable(RuntimeError):
    """A decode graph could not be captured or replayed.  The step it was asked for has not run, and the cache
    manager's books are as they were before the call: the caller can run the same entries eagerly."""


def buckets_for(max_running: int) -> List[int]:
    """1, 2, 4, ... and ``max_running`` itself (reference: buckets(7) = [1, 2, 4, 7])."""
    out, b = [], 1
    while b < max_running:
        out.append(b)
        b *= 2
    out.append(max_running)
    return out


def kv_buckets_for(max_seq_len: int, smallest: int = 512) -> List[int]:
    """Bounds on the longest sequence of a step: 512, 1024, ... and ``max_seq_len`` itself.  A graph is
    captured per bound, so that the attention grid fits the lengths it actually meets."""
    out, b = [], smallest
    while b < max_seq_len:
        out.append(b)
        b *= 2
    out.append(max_seq_len)
    return out


class _Bucket:
    def __init__(self, size, kv_bound, meta, host, offsets, ctx, caches, pinned):
        self.size = size
        self.kv_bound = kv_bound
        self.meta = meta          # device int32 buffer, fixed address
        self.host = host          # host mirror that is filled and copied over (a numpy view of `pinned`)
        self.pinned = pinned
        self.copied = None        # event after the last copy of the mirror to the device
        self.rows = {}            # (group, row) -> what the mirror's block-table row holds: (request, table version) or "pad"
        self.offsets = offsets
        self.ctx = ctx
        self.caches = caches
        self.graph = None
        self.logits = None


class GraphedDecode:
    def __init__(self, engine):
        # no reference to the engine itself is kept: engine and graphs would form a cycle, and graphs that
        # only the cycle collector frees may be destroyed while another engine is capturing, which HIP refuses
        self.runner = engine.runner
        self.cache = engine.cache
        self.device = engine.device
        self.max_seq_len = engine.cfg.max_seq_len
        self.width = engine.cfg.pages_per_request()
        self.buckets = buckets_for(engine.cfg.max_running)
        self.kv_buckets = kv_buckets_for(self.max_seq_len)
        self._made: Dict[tuple, _Bucket] = {}
        self.replays = 0
        if self.device.type != "cuda":
            raise RuntimeError("graph replay needs the GPU")

    # -- which steps ---------------------------------------------------------------
    def can_run(self, entries: List[StepEntry]) -> bool:
        """A step can be replayed if every request brings one token and wants its logits.  (A prompt's portion of
        one token that is not its last brings one token too, but wants nothing: such a step runs eagerly.)"""
        return 0 < len(entries) <= self.buckets[-1] and all(
            len(e.tokens) == 1 and list(e.want) == [0] and not e.extra for e in entries)

    def bucket_of(self, rows: int) -> int:
        return next(b for b in self.buckets if b >= rows)

    # -- buffers ---------------------------------------------------------------------
    def kv_bucket_of(self, longest: int) -> int:
        return next(b for b in self.kv_buckets if b >= longest)

    def _make(self, size: int, kv_bound: int) -> _Bucket:
        n_groups = len(self.cache.groups)
        sizes = [size, size, size, size + 1, size, size, size] + [size * self.width] * n_groups + [size, size]
        offsets = [0]
        for s in sizes:
            offsets.append(offsets[-1] + s)
        # the host mirror is pinned, so that the copy to the device needs no staging and does not wait
        pinned = torch.zeros(offsets[-1], dtype=torch.int32, pin_memory=True)
        host = pinned.numpy()
        meta = torch.zeros(offsets[-1], dtype=torch.int32, device=self.device)
        part = lambda i: meta[offsets[i]:offsets[i + 1]]
        ctx = StepContext(
            n_tokens=size, n_seqs=size, token_ids=part(0), positions=part(1), seq_of_token=part(2),
            cu_q=part(3), kv_len=part(4), state_slots=part(5), logit_rows=part(6), n_logit_rows=size,
            max_q_len=1, max_kv_len=kv_bound, kernels=self.runner.kernels,
            n_decode_seqs=size, q_lens=[1] * size, kv_bound=kv_bound)
        ctx.block_tables = [part(7 + g).view(size, self.width) for g in range(n_groups)]
        caches = self.cache.layer_caches(ctx.block_tables)
        bucket = _Bucket(size, kv_bound, meta, host, offsets, ctx, caches, pinned)
        bucket.moved = (part(7 + n_groups), part(8 + n_groups))   # rows of this step, rows of the tokens on the device
        return bucket

    def _fill(self, b: _Bucket, entries: List[StepEntry], device_tokens=None) -> None:
        """Takes this step's pages and writes the step's metadata (padding included) into the buffers.  Entries
        with ``token_from`` take their token id from that row of ``device_tokens`` (int32, on the device)."""
        size, off, host = b.size, b.offsets, b.host
        cache = self.cache
        if b.copied is not None:
            b.copied.synchronize()   # the last copy has read the mirror (long done, unless nobody read that step's result)
        tok, pos, sot, cu, kvl, slots, rows = (host[off[i]:off[i + 1]] for i in range(7))
        if not b.rows:   # first fill: what never changes
            sot[:] = np.arange(size)
            cu[:] = np.arange(size + 1)
            rows[:] = np.arange(size)
        n = len(entries)
        starts = []
        try:
            for e in entries:
                starts.append(cache.extend(e.req, 1))
        except Exception:
            # a request that found no page (replay without promises): the ones before it give theirs back, so
            # that the books are as they were before the call
            for e in entries[:len(starts)]:
                cache.retract(e.req, 1)
            raise
        tok[:n] = [e.tokens[0] for e in entries]
        pos[:n] = starts
        kvl[:n] = pos[:n] + 1
        slots[:n] = [cache.slot(e.req) for e in entries]
        tok[n:] = 0           # padding rows: token 0 at position 0 of the scratch page and slot
        pos[n:] = 0
        kvl[n:] = 1
        slots[n:] = cache.slots.scratch_slot
        # block tables: a row is rewritten only if it held another request or the request's table has changed
        for g, grp in enumerate(cache.groups):
            for s in range(size):
                base = off[7 + g] + s * self.width
                if s < len(entries):
                    req = entries[s].req
                    holds = (req, grp.versions[req])
                    if b.rows.get((g, s)) != holds:
                        row = grp.tables[req]
                        host[base:base + len(row)] = row
                        host[base + len(row):base + self.width] = -1
                        b.rows[(g, s)] = holds
                elif b.rows.get((g, s)) != "pad":
                    host[base:base + self.width] = grp.scratch_page
                    b.rows[(g, s)] = "pad"
        moved = [(s, e.token_from) for s, e in enumerate(entries) if e.token_from is not None]
        if moved:
            n_groups = len(cache.groups)
            dst, src = (host[off[7 + n_groups + i]:off[8 + n_groups + i]] for i in range(2))
            dst[:len(moved)] = [s for s, _ in moved]
            src[:len(moved)] = [r for _, r in moved]
        b.meta.copy_(b.pinned, non_blocking=True)
        if moved:
            self.runner.kernels.place_tokens(b.ctx.token_ids, b.moved[0][:len(moved)], device_tokens,
                                             b.moved[1][:len(moved)])
        if b.copied is None:
            b.copied = torch.cuda.Event()
        b.copied.record()

    # -- capture and replay -----------------------------------------------------------
    @torch.no_grad()
    def capture(self, size: int, kv_bound: int) -> _Bucket:
        b = self._make(size, kv_bound)
        self._fill(b, [])  # padding rows only: they touch the scratch page and slot
        model = self.runner.model
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        # what these runs launch is what every replay will launch: worth choosing library algorithms by measurement
        settle = getattr(self.runner.kernels, "recurring_shapes", contextlib.nullcontext)
        with torch.cuda.stream(side), settle():
            for _ in range(3):
                model.forward(b.ctx, b.caches)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()
        gc.disable()   # no destructor of an older graph may run while the stream is capturing
        try:
            with settle(), torch.cuda.graph(graph):   # records the algorithms the runs above settled on
                b.logits = model.forward(b.ctx, b.caches)
        finally:
            if collecting:
                gc.enable()
        b.graph = graph
        self._made[(size, kv_bound)] = b
        return b

    def capture_all(self, kv_bounds=None) -> None:
        """Captures every batch bucket for the given length bounds (default: the largest only; the
        others are captured when a step first needs them)."""
        for kv_bound in (kv_bounds or self.kv_buckets[-1:]):
            for size in self.buckets:
                if (size, kv_bound) not in self._made:
                    self._capture_or_give_up(size, kv_bound)

    def _capture_or_give_up(self, size: int, kv_bound: int) -> _Bucket:
        try:
            return self.capture(size, kv_bound)
        except Exception as exc:     # capture is fragile: memory for a private pool, a library that cannot be recorded
            raise GraphUnavailable(f"capture of the graph for {size} rows and {kv_bound} positions failed") from exc

    @torch.no_grad()
    def run(self, entries: List[StepEntry], device_tokens=None) -> torch.Tensor:
        """Logits ``[len(entries), vocab]`` of a step of single tokens.  An entry with ``token_from`` holds a
        placeholder; its token id is that row of ``device_tokens`` (int32, on the device): the sampler's output of
        the step before, which the host need not have read yet.  Raises ``GraphUnavailable``, with nothing
        booked, if the graph cannot be captured or replayed."""
        self.runner._check(entries)
        if not self.can_run(entries):
            raise ValueError("a replayed step takes one token per request and returns its logits")
        for e in entries:
            if e.token_from is not None and (device_tokens is None or device_tokens.dtype != torch.int32
                                             or not 0 <= e.token_from < device_tokens.numel()):
                raise ValueError("an entry takes its token from a row of int32 device_tokens that was not given")
        size = self.bucket_of(len(entries))
        longest = max(self.cache.lengths[e.req] for e in entries) + 1
        kv_bound = self.kv_bucket_of(longest)
        b = self._made.get((size, kv_bound)) or self._capture_or_give_up(size, kv_bound)
        self._fill(b, entries, device_tokens)     # takes the step's pages: from here on the step is booked
        try:
            b.graph.replay()
        except Exception as exc:
            for e in entries:
                self.cache.retract(e.req, 1)
            raise GraphUnavailable(f"replay of the graph for {size} rows and {kv_bound} positions failed") from exc
        self.replays += 1
        return b.logits[:len(entries)]
