"""Weights from safetensors, bound by tensor name.

Discovery follows the reference (``loader.py:179-203``): a
``model.safetensors.index.json`` with a ``weight_map``, else a single
``model.safetensors``.  Where the reference raises a ``KeyError`` for the first
name it misses (``loader.py:218-226``), this loader compares the whole set of
names and shapes with what the model's parts want and raises ONE ``WeightError``
that lists every missing tensor, every unexpected tensor and every wrong shape.

Dtypes.  A tensor stored in bfloat16 (or float16) is kept in bfloat16 when the
engine computes in bfloat16 and widened (exactly) when it computes in float32.
A tensor stored in float32 stays float32 in both modes; integer tables become
int32; small vectors (norm gains) are held in float32 whatever their storage.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable, Mapping, Tuple

import torch

from ..parts.plan import TensorSpec


class WeightError(ValueError):
    """The checkpoint does not hold what the model wants; lists all differences."""

    def __init__(self, missing, unexpected, wrong_shape, where="", differing=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.differing = list(differing)   # (name, the tensor it should repeat): stored twice with different values
        lines = [f"checkpoint {where} does not match the model:".replace("  ", " ")]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, wanted {list(want)}" for n, got, want in self.wrong_shape))
        if self.differing:
            lines.append(f"  stored twice with different values ({len(self.differing)}): " + ", ".join(
                f"{n} is not equal to {other}, which the configuration says it shares" for n, other in self.differing))
        super().__init__("\n".join(lines))


def _shard_map(folder: Path) -> Dict[str, Path]:
    """Tensor name -> file that holds it."""
    from safetensors import safe_open

    index = folder / "model.safetensors.index.json"
    single = folder / "model.safetensors"
    names: Dict[str, Path] = {}
    if index.is_file():
        with open(index) as f:
            weight_map = json.load(f)["weight_map"]
        for name, shard in weight_map.items():
            path = folder / shard
            if not path.is_file():
                raise FileNotFoundError(f"{index} names shard {shard}, which is not in {folder}")
            names[name] = path
    elif single.is_file():
        with safe_open(str(single), framework="pt") as f:
            for name in f.keys():
                names[name] = single
    else:
        raise FileNotFoundError(f"no model.safetensors or model.safetensors.index.json in {folder}")
    return names


def target_dtype(stored: torch.dtype, role: str, compute: torch.dtype) -> torch.dtype:
    if role == "table" or not stored.is_floating_point:
        return torch.int32
    if role == "vector" or stored == torch.float32 or stored == torch.float64:
        return torch.float32
    return compute  # bfloat16 / float16 storage follows the engine


def check_names_and_shapes(found: Mapping[str, Tuple[int, ...]], expected: Mapping[str, TensorSpec],
                           ignore_suffixes: Iterable[str] = (), where: str = "",
                           duplicates: Mapping[str, str] = {}) -> None:
    ignore = tuple(ignore_suffixes)
    missing = [n for n in expected if n not in found]
    unexpected = [n for n in found if n not in expected and n not in duplicates and not (ignore and n.endswith(ignore))]
    wrong = [(n, tuple(found[n]), tuple(expected[n].shape)) for n in expected
             if n in found and tuple(found[n]) != tuple(expected[n].shape)]
    wrong += [(n, tuple(found[n]), tuple(expected[other].shape)) for n, other in duplicates.items()
              if n in found and n not in expected and other in expected
              and tuple(found[n]) != tuple(expected[other].shape)]
    if missing or unexpected or wrong:
        raise WeightError(sorted(missing), sorted(unexpected), wrong, where)


def load_weights(folder, expected: Mapping[str, TensorSpec], device, compute_dtype: torch.dtype,
                 ignore_suffixes: Iterable[str] = ("rotary_emb.inv_freq",),
                 duplicates: Mapping[str, str] = {}) -> Dict[str, torch.Tensor]:
    """Reads the tensors named in ``expected`` from a model folder onto ``device``.

    ``duplicates`` maps names a checkpoint may hold beside the expected ones to the expected tensor each must
    repeat (a tied model stored with its ``lm_head.weight``: the reference takes such a file,
    ``model/llama.py:147-154``).  A duplicate equal to its tensor is passed over; one that differs is an error,
    since the engine would compute with one of the two and the file means the other."""
    from safetensors import safe_open

    folder = Path(folder)
    shards = _shard_map(folder)
    handles = {}
    try:
        for path in set(shards.values()):
            handles[path] = safe_open(str(path), framework="pt")
        shapes = {name: tuple(handles[path].get_slice(name).get_shape()) for name, path in shards.items()}
        duplicates = {n: other for n, other in duplicates.items() if n not in expected and other in expected}
        check_names_and_shapes(shapes, expected, ignore_suffixes, where=str(folder), duplicates=duplicates)
        differing = [(n, other) for n, other in sorted(duplicates.items()) if n in shards and not torch.equal(
            handles[shards[n]].get_tensor(n).float(), handles[shards[other]].get_tensor(other).float())]
        if differing:
            raise WeightError((), (), (), str(folder), differing)
        out: Dict[str, torch.Tensor] = {}
        for name, spec in expected.items():
            t = handles[shards[name]].get_tensor(name)
            out[name] = t.to(device=device, dtype=target_dtype(t.dtype, spec.role, compute_dtype)).contiguous()
        return out
    finally:
        for h in handles.values():
            close = getattr(h, "__exit__", None)
            if close is not None:
                close(None, None, None)
