"""Dense gated feed-forward (reference: ``ops/mlp.py:87-128``).

``y = (silu(h Wg^T) * (h Wu^T)) Wd^T``.  Gate and up are stacked into one
``[2I, H]`` matrix at load (reference: ``ops/mlp.py:104``) so one product gives
both; ``silu(g) * u`` is computed in float32 and rounded once (reference:
``kernels/swiglu_kernel.py:142-150``).
"""

from __future__ import annotations

import torch

from .plan import TensorSpec
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU:
    """params: hidden_size, intermediate_size."""

    takes_scaled_rows = True   # the input goes to ``gated_linear`` only

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.env = env
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self):
        return {
            "gate": TensorSpec((self.inter, self.hidden)),
            "up": TensorSpec((self.inter, self.hidden)),
            "down": TensorSpec((self.hidden, self.inter)),
        }

    def bind(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate"], tensors["up"]], dim=0).contiguous()
        self.w_down = tensors["down"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:   # the kernels may keep a copy of their own of a weight whose product is left pending
            prepare(self.w_down)

    def plain_form(self):
        """What this feed-forward is, as plain data, for kernels that can run a whole block in one call (None for
        a subclass with a forward of its own: it is no longer what this form describes)."""
        if type(self).forward is not SwiGLU.forward:
            return None
        return {"kind": "swiglu", "w_gate_up": self.w_gate_up, "w_down": self.w_down, "hidden": self.hidden,
                "inter": self.inter}

    def forward(self, h, ctx):
        k = self.env.kernels
        a = k.gated_linear(h, self.w_gate_up)   # the activation is fused into the product where a kernel has it
        return k.pending_linear(a, self.w_down)   # the norm after it may have it added into the residual
