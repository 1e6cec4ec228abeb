"""Rotary position encoding with llama3 frequency scaling.

Frequencies (reference: ``ops/rope.py:95-118``): ``inv_freq_i = 1 / theta^(2i/d)``
for ``i = 0 .. d/2-1`` in float32.  With ``rope_type == "llama3"`` each frequency
is rescaled by its wavelength (reference: ``ops/rope.py:120-155``): unchanged below
``original/high_freq_factor``, divided by ``factor`` above
``original/low_freq_factor``, interpolated in between; that loop runs in Python
floats on the float32 values, as the reference's does.  Angles are
``float32(position) * inv_freq`` and the cos/sin tables stay float32.  The
rotation itself pairs element ``i`` with ``i + d/2`` (reference:
``ops/rope.py:167-182``) and is applied by the kernel that also writes the cache.
"""

from __future__ import annotations

import math

import torch

from .registry import register_position_encoding


def rotary_inv_freq(rotary_dim: int, theta: float, scaling=None) -> torch.Tensor:
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / (theta ** (idx / rotary_dim))
    if scaling is None or scaling.get("rope_type", "default") != "llama3":
        return inv_freq
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    original = float(scaling["original_max_position_embeddings"])
    low_wavelen = original / low
    high_wavelen = original / high
    scaled = []
    for f in inv_freq.tolist():
        wavelen = 2 * math.pi / f
        if wavelen < high_wavelen:
            scaled.append(f)
        elif wavelen > low_wavelen:
            scaled.append(f / factor)
        else:
            smooth = (original / wavelen - low) / (high - low)
            scaled.append((1 - smooth) * f / factor + smooth * f)
    return torch.tensor(scaled, dtype=torch.float32)


@register_position_encoding("rope")
class RotaryEncoding:
    """params: rotary_dim, theta, scaling (dict or None)."""

    def __init__(self, params, env):
        self.rotary_dim = int(params["rotary_dim"])
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {self.rotary_dim}")
        self.theta = float(params["theta"])
        self.scaling = params.get("scaling")
        self.max_positions = int(env.max_positions)
        self.device = env.device
        self._tables = None

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def tables(self):
        """(cos, sin), each float32 ``[max_positions, rotary_dim/2]``, on the device."""
        if self._tables is None:
            inv_freq = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling)
            pos = torch.arange(self.max_positions, dtype=torch.float32)
            angles = torch.outer(pos, inv_freq)
            self._tables = (angles.cos().to(self.device).contiguous(),
                            angles.sin().to(self.device).contiguous())
        return self._tables


@register_position_encoding("none")
class NoPositionEncoding:
    rotary_dim = 0

    def __init__(self, params, env):
        pass

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def tables(self):
        return None, None
