"""Registries of part kinds: mixers, feed-forwards, norms, position encodings, blocks, embeddings, heads.

A part class is registered under a ``kind``; a ``PartSpec`` names that kind.  A
test or a user package adds a part with one ``register_*`` call and without a
change to this package's files.

Interfaces (``env`` is a ``BuildEnv``; ``ctx`` a ``StepContext``):

* every part: ``__init__(self, params: dict, env)``,
  ``weight_specs() -> dict[str, TensorSpec]`` (own tensor names),
  ``bind(tensors: dict[str, Tensor])``.
* mixer: ``cache_need() -> PagedKVNeed | None``, ``state_need() -> StateNeed | None``,
  ``forward(h, ctx, cache) -> Tensor[N, hidden]``; ``cache`` is the ``LayerCache``
  of this run of the layer (pages, block table, state rows).
* feed-forward: ``forward(h, ctx) -> Tensor[N, hidden]``.
* norm: ``forward(stream, rows=None) -> Tensor``: adds the stream's pending
  delta into its 32-bit residual and returns the normalised rows.
* position encoding: whatever its mixer consumes; the rotary kind gives
  ``tables(device) -> (cos, sin)`` indexed by absolute position.
* block: ``__init__(self, **parts)`` with the names it gives its parts as keyword arguments (the pre-norm
  block: ``mixer, feed_forward, mixer_norm, feed_forward_norm``; a ``LayerSpec`` names the parts of its
  layer under those names), ``forward(stream, ctx, cache) -> None``.
* embedding: ``forward(ctx) -> Tensor[N, hidden]`` float32, the residual stream's start.
* head: ``forward(h) -> Tensor[rows, vocab]`` float32 logits; a head that can use the embedding's
  matrix has ``share_embedding(embedding)``, called before ``bind`` when its params say ``tied``.
"""

from __future__ import annotations

from typing import Callable, Dict


class _Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, type] = {}

    def register(self, kind: str, cls=None, *, replace: bool = False):
        def put(c):
            if kind in self._items and not replace:
                raise ValueError(f"{self.what} kind {kind!r} is already registered")
            self._items[kind] = c
            return c
        return put if cls is None else put(cls)

    def unregister(self, kind: str) -> None:
        self._items.pop(kind, None)

    def get(self, kind: str):
        try:
            return self._items[kind]
        except KeyError:
            raise KeyError(
                f"unknown {self.what} kind {kind!r}; known: {', '.join(sorted(self._items)) or '(none)'}"
            ) from None

    def kinds(self):
        return sorted(self._items)


MIXERS = _Registry("mixer")
FEED_FORWARDS = _Registry("feed-forward")
NORMS = _Registry("norm")
POSITION_ENCODINGS = _Registry("position encoding")
BLOCKS = _Registry("block")
EMBEDDINGS = _Registry("embedding")
HEADS = _Registry("head")

register_mixer: Callable = MIXERS.register
register_feed_forward: Callable = FEED_FORWARDS.register
register_norm: Callable = NORMS.register
register_position_encoding: Callable = POSITION_ENCODINGS.register
register_block: Callable = BLOCKS.register
register_embedding: Callable = EMBEDDINGS.register
register_head: Callable = HEADS.register
