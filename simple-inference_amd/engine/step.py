"""The step function: one batch of (request, its next tokens) through the model.

A batch holds, for each of its requests, a run of that request's next tokens:
a whole prompt, a portion of one cut anywhere, or one decoded token; all runs
of a step form one flat batch.  The step runs only the tokens it is given,
against the pages that earlier steps wrote, writes these tokens' keys and values,
and returns float32 logits at the places asked for.

The reference has two runners instead, which it calls back to back and never
mixes: whole right-padded prompts (``serving/prefill.py:60-76``) and single
decoded tokens (``serving/paged_decoder.py:364-408``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..parts.context import StepContext
from ..parts.model import DecoderModel


@dataclass
class StepEntry:
    req: int                         # the request's id in the cache manager
    tokens: Sequence[int]            # its next tokens, in order
    want: Sequence[int] = field(default_factory=list)  # places among ``tokens`` whose logits are wanted
    token_from: Optional[int] = None  # the one token is row ``token_from`` of the step's ``device_tokens``; ``tokens`` holds a placeholder
    extra: Optional[dict] = None     # further integers per token, by name (e.g. a second position axis): each len(tokens) long


class StepRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, kernels, device, max_positions: int):
        self.model = model
        self.cache = cache
        self.kernels = kernels
        self.device = torch.device(device)
        self.max_positions = max_positions
        self.vocab_size = model.vocab_size
        self._stages, self._stage_turn = [], -1

    def _staging(self, size: int):
        """Host memory for a step's metadata: on a GPU one of a few pinned buffers used in turn (each free again when
        the copy out of it has run), so that the host can lay out the next step while earlier ones are still queued."""
        if self.device.type != "cuda":
            return np.empty(size, dtype=np.int32), None
        self._stage_turn = (self._stage_turn + 1) % 3
        if len(self._stages) <= self._stage_turn:
            self._stages.append(None)
        stage = self._stages[self._stage_turn]
        if stage is None or stage[0].numel() < size:
            pinned = torch.empty(max(size, 4096, 2 * (stage[0].numel() if stage else 0)), dtype=torch.int32, pin_memory=True)
            stage = self._stages[self._stage_turn] = (pinned, torch.cuda.Event(), [False])
        pinned, copied, used = stage
        if used[0]:
            copied.synchronize()    # long done, unless the host is three steps ahead
        used[0] = True
        return pinned.numpy()[:size], (pinned, copied)

    def _check(self, entries: List[StepEntry]) -> dict:
        """Raises for entries that cannot run; returns every request's token ids as an array."""
        seen = set()
        arrays = {}
        extra_keys = {key for e in entries if e.extra for key in e.extra}
        for e in entries:
            for key in extra_keys:
                if e.extra is None or key not in e.extra or len(e.extra[key]) != len(e.tokens):
                    raise ValueError(f"request {e.req}: per-token values {key!r} must be given for every request of "
                                     f"the step, one per token")
            if e.req in seen:
                raise ValueError(f"request {e.req} appears twice in one step")
            seen.add(e.req)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req} brings no tokens")
            if e.req not in self.cache.lengths:
                raise KeyError(f"request {e.req} is not admitted to the cache")
            if self.cache.lengths[e.req] + len(e.tokens) > self.max_positions:
                raise ValueError(
                    f"request {e.req} would reach position {self.cache.lengths[e.req] + len(e.tokens)}, "
                    f"beyond the engine's {self.max_positions}")
            ids = arrays[e.req] = np.asarray(e.tokens)      # checked as a whole: a prompt portion has thousands
            if ids.dtype.kind not in "iu":
                raise ValueError(f"the token ids of request {e.req} are not integers ({ids.dtype})")
            if int(ids.min()) < 0 or int(ids.max()) >= self.vocab_size:
                t = next(int(t) for t in ids if not 0 <= int(t) < self.vocab_size)
                raise ValueError(f"token id {t} of request {e.req} is outside [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"wanted place {w} of request {e.req} is outside its {len(e.tokens)} tokens")
        return arrays

    def build_context(self, entries: List[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> StepContext:
        """Takes the pages the step needs and lays its metadata out on the device.  Entries with ``token_from``
        get their token id from ``device_tokens`` (int32, on the device), by a copy on the device."""
        token_arrays = self._check(entries)
        from_device = [e for e in entries if e.token_from is not None]
        if from_device:
            if device_tokens is None or device_tokens.dtype != torch.int32:
                raise ValueError("entries take their tokens from the device, but no int32 device_tokens were given")
            for e in from_device:
                if len(e.tokens) != 1 or not 0 <= e.token_from < device_tokens.numel():
                    raise ValueError(f"request {e.req}: a token from the device is one token, at a row of device_tokens")
        cache = self.cache
        n_seqs = len(entries)
        # Sequences that bring one token go first: the kernels treat them apart from longer runs.
        order = sorted(range(n_seqs), key=lambda i: len(entries[i].tokens) != 1)
        seqs = [entries[i] for i in order]
        q_lens = [len(e.tokens) for e in seqs]
        n_decode = sum(1 for n in q_lens if n == 1)
        n_tokens = sum(q_lens)
        starts = [cache.extend(e.req, len(e.tokens)) for e in seqs]
        n_groups = len(cache.groups)
        width = max(1, cache.max_table_len([e.req for e in seqs]))
        n_rows = sum(len(e.want) for e in entries)

        n_moved = len(from_device)
        extra_keys = sorted({key for e in seqs if e.extra for key in e.extra})
        sizes = [n_tokens, n_tokens, n_tokens, n_seqs + 1, n_seqs, n_seqs, max(n_rows, 1)] + \
                [n_seqs * width] * n_groups + [n_moved, n_moved] + [n_tokens] * len(extra_keys)
        offsets = np.concatenate([[0], np.cumsum(sizes)])
        host, staged = self._staging(int(offsets[-1]))
        tok, pos, sot, cu, kvl, slots, rows = (host[offsets[i]:offsets[i + 1]] for i in range(7))
        cu[0] = 0
        rows[:] = 0
        t = 0
        first_token = {}
        for s, e in enumerate(seqs):
            n = q_lens[s]
            tok[t:t + n] = token_arrays[e.req]
            pos[t:t + n] = np.arange(starts[s], starts[s] + n, dtype=np.int32)
            sot[t:t + n] = s
            first_token[e.req] = t
            t += n
            cu[s + 1] = t
            kvl[s] = starts[s] + n
            slots[s] = cache.slot(e.req)
        r = 0
        for e in entries:  # logits come back in the order of the entries as given
            for w in e.want:
                rows[r] = first_token[e.req] + int(w)
                r += 1
        for g in range(n_groups):
            tab = host[offsets[7 + g]:offsets[8 + g]].reshape(n_seqs, width)
            tab[:] = -1
            for s, e in enumerate(seqs):
                row = cache.table(g, e.req)
                tab[s, :len(row)] = row

        if n_moved:
            dst, src = (host[offsets[7 + n_groups + i]:offsets[8 + n_groups + i]] for i in range(2))
            dst[:] = [first_token[e.req] for e in from_device]
            src[:] = [e.token_from for e in from_device]

        for i, key in enumerate(extra_keys):
            col = host[offsets[9 + n_groups + i]:offsets[10 + n_groups + i]]
            t = 0
            for e in seqs:
                col[t:t + len(e.tokens)] = e.extra[key]
                t += len(e.tokens)

        if staged is None:
            dev = torch.from_numpy(host).to(self.device)
        else:   # from pinned memory, without waiting for the steps that are still queued in front of this one
            pinned, copied = staged
            dev = torch.empty(host.size, dtype=torch.int32, device=self.device)
            dev.copy_(pinned[:host.size], non_blocking=True)
            copied.record()
        part = lambda i: dev[int(offsets[i]):int(offsets[i + 1])]
        if n_moved:
            self.kernels.place_tokens(part(0), part(7 + n_groups), device_tokens, part(8 + n_groups))
        ctx = StepContext(
            n_tokens=n_tokens, n_seqs=n_seqs,
            token_ids=part(0), positions=part(1), seq_of_token=part(2), cu_q=part(3), kv_len=part(4),
            state_slots=part(5), logit_rows=part(6)[:n_rows] if n_rows else None, n_logit_rows=n_rows,
            max_q_len=max(q_lens), max_kv_len=int(kvl.max()), kernels=self.kernels,
            n_decode_seqs=n_decode, q_lens=q_lens,
            max_run_kv_len=int(kvl[n_decode:].max()) if n_decode < n_seqs else 0,
        )
        ctx.block_tables = [part(7 + g).view(n_seqs, width) for g in range(n_groups)]
        ctx.extra = {key: part(9 + n_groups + i) for i, key in enumerate(extra_keys)}
        return ctx

    @torch.no_grad()
    def run(self, entries: List[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Runs one step; returns float32 logits ``[wanted, vocab]`` in the order of entries and wants."""
        ctx = self.build_context(entries, device_tokens)
        caches = self.cache.layer_caches(ctx.block_tables)
        return self.model.forward(ctx, caches)
