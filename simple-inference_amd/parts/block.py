"""The arrangement of parts in a layer.

Pre-norm (reference: ``model/block.py:135-147``):
``x += mixer(norm1(x))``; ``x += feed_forward(norm2(x))``.  Each add is carried
as the stream's pending delta and summed into the float32 residual by the norm
that follows (the next layer's, or the model's last norm).
"""

from __future__ import annotations

from .registry import register_block


@register_block("prenorm")
class PreNormBlock:
    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm
        self.plain_forms = None   # kept by kernels that run the block in one call: what they made of the parts

    def plain_form(self):
        """What this block is, as plain data, for kernels that can make all of its launches in one call: its kind
        (the order in which the parts run is this file's affair: the docstring above) and what each part says it is
        (its own ``plain_form``; None for a part that has none, and such a block goes part by part)."""
        if type(self).forward is not PreNormBlock.forward:
            return None
        form = lambda part: getattr(part, "plain_form", lambda: None)()
        return {"kind": "prenorm", "mixer_norm": form(self.mixer_norm), "mixer": form(self.mixer),
                "feed_forward_norm": form(self.feed_forward_norm), "feed_forward": form(self.feed_forward)}

    def forward(self, stream, ctx, cache):
        # Kernels that can make all of a block's launches in one call are shown the block (they look at what it and
        # its parts say they are, ``plain_form``, and take it or leave it); else part by part.
        whole = getattr(ctx.kernels, "prenorm_block", None)
        if whole is not None and whole(self, stream, ctx, cache):
            return
        h = _normed(self.mixer_norm, self.mixer, stream)
        stream.delta = self.mixer.forward(h, ctx, cache)
        h = _normed(self.feed_forward_norm, self.feed_forward, stream)
        stream.delta = self.feed_forward.forward(h, ctx)


def _normed(norm, consumer, stream):
    """The norm's rows for ``consumer``.  A norm that ``gives_scaled_rows`` may leave the division by the root mean
    square to a consumer that ``takes_scaled_rows`` (one that hands its input to the kernels' products only)."""
    if getattr(norm, "gives_scaled_rows", False) and getattr(consumer, "takes_scaled_rows", False):
        return norm.forward(stream, scaled_ok=True)
    return norm.forward(stream)
