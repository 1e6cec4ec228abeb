"""Token embedding and output head (reference: ``ops/embedding.py:49-92``).

The embedding gathers rows of ``[V, H]`` into the float32 residual.  The head is
``logits = h E^T``; tied, it uses the embedding's storage (reference:
``ops/embedding.py:78-86``); untied, it has a matrix of its own, which the
reference mishandles by overwriting the embedding (``model/llama.py:147-154``).
Logits leave the head as float32.
"""

from __future__ import annotations

from .plan import TensorSpec
from .registry import register_embedding, register_head


@register_embedding("embedding")
class TokenEmbedding:
    def __init__(self, params, env):
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.env = env
        self.weight = None

    def weight_specs(self):
        return {"weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, ctx):
        return self.env.kernels.embed(ctx.token_ids, self.weight)


@register_head("head")
class OutputHead:
    """params: vocab_size, hidden_size, tied."""

    def __init__(self, params, env):
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.tied = bool(params["tied"])
        self.env = env
        self.embedding = None
        self._weight = None

    def share_embedding(self, embedding) -> None:
        """A tied head multiplies by the embedding's matrix: the same storage, not a copy."""
        if (embedding.vocab, embedding.hidden) != (self.vocab, self.hidden):
            raise ValueError(f"a head of {self.vocab} x {self.hidden} cannot share an embedding of "
                             f"{embedding.vocab} x {embedding.hidden}")
        self.embedding = embedding

    def weight_specs(self):
        return {} if self.tied else {"weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        if not self.tied:
            self._weight = tensors["weight"]
        elif self.embedding is None:
            raise ValueError("a tied head was given no embedding to share")

    @property
    def weight(self):
        return self.embedding.weight if self.tied else self._weight

    def forward(self, h):
        return self.env.kernels.linear(h, self.weight, out_float32=True)
