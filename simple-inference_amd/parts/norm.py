"""Root-mean-square norm (reference: ``ops/rmsnorm.py:41-46``, ``kernels/rmsnorm_kernel.py:105-113``).

``y = x * rsqrt(mean(x^2) + eps) * w`` with the statistic, the normalisation and
the gain in float32 and one rounding to the compute dtype, as the reference's
fused kernel does.  The add of the pending residual delta is fused in front.
"""

from __future__ import annotations

from .plan import TensorSpec
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm:
    def __init__(self, params, env):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.env = env
        self.weight = None

    def weight_specs(self):
        return {"weight": TensorSpec((self.size,), "vector")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    gives_scaled_rows = True

    def plain_form(self):
        """What this norm is, as plain data, for kernels that can run a whole block in one call (None for a
        subclass with a forward of its own: it is no longer what this form describes)."""
        if type(self).forward is not RMSNorm.forward:
            return None
        return {"kind": "rmsnorm", "weight": self.weight, "eps": self.eps, "size": self.size}

    def forward(self, stream, rows=None, scaled_ok=False):
        """Adds ``stream.delta`` into ``stream.residual`` and returns the normed rows.

        With ``rows`` (int32 indices) only those rows are computed and the residual
        is left as it was: that form ends a forward pass.

        ``scaled_ok``: the caller also takes the rows undivided by their root mean square (the kernels'
        ``ScaledRows``).  Then a delta that is a product not yet computed is computed into the residual by the
        product's own kernel, and the product after the norm divides: the norm has no kernel of its own.
        """
        k = self.env.kernels
        if scaled_ok and rows is None and hasattr(stream.raw_delta, "compute") and hasattr(k, "linear_into_residual"):
            out = k.linear_into_residual(stream.raw_delta, stream.residual, self.weight, self.eps)
            stream.delta = None
            return out
        out = self.env.kernels.add_rmsnorm(
            stream.residual, stream.delta, self.weight, self.eps, self.env.dtype, rows)
        if rows is None:
            stream.delta = None
        return out
