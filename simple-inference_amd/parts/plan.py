"""The data that describes a model: which parts each layer has and how layers run.

A ``ModelPlan`` is plain data.  An architecture's ``build_plan`` writes it from
its configuration; ``DecoderModel`` builds the parts it names.  Nothing in a plan
refers to a concrete architecture: a part is named by its ``kind`` (a key of the
part registries), its sizes and constants are in ``params``, and ``weights`` maps
the part's own tensor names to the names in the checkpoint.

* Layers may differ from one another: every ``LayerSpec`` names its own block kind and
  the parts that kind arranges (for the pre-norm block: a mixer, a feed-forward and
  their two norms; another block kind may take a third norm, no feed-forward, or
  whatever names it defines).
* ``order`` lists layer indices in the order they run.  A layer may be named
  twice (each run keeps a cache of its own), and a mixer may read the cache
  that another layer's latest run wrote (``params["kv_from_layer"]``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    weights: Dict[str, str] = field(default_factory=dict)
    role: str = ""     # in a layer: which registry ``kind`` is looked up in ("mixer", "feed_forward", "norm")


ROLES = ("mixer", "feed_forward", "norm")


@dataclass
class LayerSpec:
    """A layer: a block kind and the named parts that this kind arranges.

    ``parts`` maps the names the block kind gives its parts (they are the keyword arguments of its constructor) to
    their specs; a spec's ``role`` says which registry its kind is looked up in.  The four arguments ``mixer``,
    ``feed_forward``, ``mixer_norm`` and ``feed_forward_norm`` are a shorter way to write the parts of the pre-norm
    block (and of any block kind that keeps those names): they are put into ``parts`` under their names, with
    their roles.  A layer has at most one part of role "mixer": the run of a layer owns one set of pages and one
    state; a layer without a mixer owns none.
    """

    mixer: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    feed_forward_norm: Optional[PartSpec] = None
    block: str = "prenorm"
    parts: Dict[str, PartSpec] = field(default_factory=dict)

    def __post_init__(self):
        short = (("mixer_norm", "norm"), ("mixer", "mixer"), ("feed_forward_norm", "norm"), ("feed_forward", "feed_forward"))
        named = dict(self.parts)
        self.parts = {}
        for name, role in short:
            spec = getattr(self, name)
            if spec is None:
                spec = named.pop(name, None)
                if spec is None:
                    continue
            elif name in named:
                raise ValueError(f"the layer names its part {name!r} twice")
            if not spec.role:
                spec.role = role
            self.parts[name] = spec
            setattr(self, name, spec)
        self.parts.update(named)
        for name, spec in self.parts.items():
            if spec.role not in ROLES:
                raise ValueError(f"part {name!r} of a layer has role {spec.role!r}; a role is one of {', '.join(ROLES)}")
        if sum(spec.role == "mixer" for spec in self.parts.values()) > 1:
            raise ValueError("a layer has at most one part of role 'mixer'")


@dataclass
class ModelPlan:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    final_norm: PartSpec
    head: PartSpec
    order: Optional[List[int]] = None  # None → every layer once, in index order
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    max_position_embeddings: Optional[int] = None
    # checkpoint names that may be stored beside the parts' tensors -> the tensor each must then be equal to
    duplicates: Dict[str, str] = field(default_factory=dict)

    def run_order(self) -> List[int]:
        order = list(range(len(self.layers))) if self.order is None else list(self.order)
        for i in order:
            if not 0 <= i < len(self.layers):
                raise ValueError(f"order names layer {i}, but the plan has {len(self.layers)} layers")
        return order


# ---------------------------------------------------------------------------
# What a part asks of the loader and of the cache manager
# ---------------------------------------------------------------------------

@dataclass(frozen=True)
class TensorSpec:
    """Shape and role of one tensor a part reads from the checkpoint.

    role "matrix": kept in the engine's compute dtype (bfloat16 or float32).
    role "vector": small gains and the like, held in float32 in both modes.
    role "table":  integers, held as int32.
    """

    shape: Tuple[int, ...]
    role: str = "matrix"


@dataclass(frozen=True)
class PagedKVNeed:
    """Keys and values in pages: all keys (``window`` None) or the last ``window``.

    A page holds, per key/value head, ``page_size`` key rows of ``head_dim`` elements and as many value rows of
    ``value_head_dim`` elements (None: the same width).  The cache manager only stores them; what a row means is
    the mixer's affair, so a mixer that caches something narrower or wider beside its keys names that width here.
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_head_dim: Optional[int] = None

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.value_head_dim is None else self.value_head_dim


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size (one row per running request).  A request's row holds ``init`` in every
    element when the request gets its slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"
    init: float = 0.0
