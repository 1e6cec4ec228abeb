"""Grouped-query attention over the paged cache (reference: ``ops/attention.py:70-228``,
serving form ``serving/paged_decoder.py:133-185``).

Order inside the mixer, as in the reference's serving path: project q, k, v (no
bias) -> rotate q and k by absolute position -> write k (rotated) and v into
the pages -> attend over the pages, the tokens just written included -> output
projection.  Query head ``h`` reads key/value head ``h // (Hq / Hkv)`` (reference:
``kernels/attention_kernel.py:108-251``).  Scores are ``(q . k) * scale`` with the
scale applied after the dot; key ``j`` is visible to a query at position ``p`` iff
``j <= p`` and, with a window ``w``, ``j > p - w``.

The three projections are stacked into one ``[(Hq + 2 Hkv) D, H]`` matrix at load.
A mixer whose ``kv_from_layer`` is set projects only q and reads the pages that
the named layer's latest run wrote.
"""

from __future__ import annotations

import torch

from .plan import PagedKVNeed, TensorSpec
from .registry import POSITION_ENCODINGS, register_mixer


def _shared_position_encoding(spec, env):
    kind = spec["kind"] if isinstance(spec, dict) else spec.kind
    params = spec["params"] if isinstance(spec, dict) else spec.params
    key = ("position", kind, repr(sorted(params.items(), key=lambda kv: kv[0])))
    if key not in env._shared:
        env._shared[key] = POSITION_ENCODINGS.get(kind)(params, env)
    return env._shared[key]


@register_mixer("attention")
class Attention:
    """params: hidden_size, num_heads, num_kv_heads, head_dim, position
    (``{"kind", "params"}``), and optionally window, scale, kv_from_layer."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        self.window = params.get("window")
        if self.window is not None:
            self.window = int(self.window)
            if self.window <= 0:
                raise ValueError(f"window must be positive, got {self.window}")
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / (self.head_dim ** 0.5)
        self.kv_from_layer = params.get("kv_from_layer")
        self.position = _shared_position_encoding(params.get("position", {"kind": "none", "params": {}}), env)
        if self.position.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head_dim {self.head_dim}")
        check = getattr(env.kernels, "check_attention_geometry", None)
        if check is not None:     # sizes the kernels refuse are refused here, when the model is built
            check(self.num_heads, self.num_kv_heads, self.head_dim)
        self.env = env
        self.w_qkv = None
        self.w_o = None

    takes_scaled_rows = True   # the input goes to ``qkv_to_cache`` only

    @property
    def writes_kv(self) -> bool:
        return self.kv_from_layer is None

    def weight_specs(self):
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        specs = {"q": TensorSpec((q, self.hidden)), "o": TensorSpec((self.hidden, q))}
        if self.writes_kv:
            specs["k"] = TensorSpec((kv, self.hidden))
            specs["v"] = TensorSpec((kv, self.hidden))
        return specs

    def bind(self, tensors):
        if self.writes_kv:
            self.w_qkv = torch.cat([tensors["q"], tensors["k"], tensors["v"]], dim=0).contiguous()
        else:
            self.w_qkv = tensors["q"].contiguous()
        self.w_o = tensors["o"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:   # the kernels may keep a copy of their own of a weight whose product is left pending
            prepare(self.w_o)

    def plain_form(self):
        """What this mixer is, as plain data, for kernels that can run a whole block in one call; None for the forms
        that only ``forward`` covers (reading another layer's keys and values)."""
        if not self.writes_kv or type(self).forward is not Attention.forward:
            return None     # a subclass with a forward of its own is no longer what this form describes
        cos, sin = self.position.tables()
        return {"kind": "paged_attention", "w_qkv": self.w_qkv, "w_o": self.w_o, "hidden": self.hidden,
                "n_heads": self.num_heads, "n_kv_heads": self.num_kv_heads, "head_dim": self.head_dim,
                "rotary_dim": self.position.rotary_dim, "cos": cos, "sin": sin, "scale": self.scale,
                "window": self.window}

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def state_need(self):
        return None

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        cos, sin = self.position.tables()
        qkv = k.qkv_to_cache(
            h, self.w_qkv, self.num_heads, self.num_kv_heads if self.writes_kv else 0, self.head_dim,
            self.position.rotary_dim, cos, sin, ctx, cache)
        out = k.paged_attention(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, ctx, cache)
        return k.pending_linear(out, self.w_o)   # the norm after it may have it added into the residual
