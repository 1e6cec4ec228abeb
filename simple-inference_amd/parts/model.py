"""A decoder built from a ``ModelPlan``: embed -> runs of layers -> norm -> head.

(Reference: ``model/llama.py:156-186``.)  This class knows no architecture.  It
builds the parts the plan names, tells the loader which tensors they want under
which checkpoint names, tells the cache manager what each run of a layer needs,
and runs a step's tokens through the layers in the plan's order.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .context import BuildEnv, LayerCache, ResidualStream, StepContext
from .plan import ModelPlan, PagedKVNeed, StateNeed, TensorSpec
from .registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS


@dataclass
class CacheLayout:
    """What the cache manager has to provide for a model.

    ``kv_groups[g]`` is the need shared by all runs in group ``g`` and
    ``kv_slabs[g]`` the number of runs that write pages of their own there.
    ``run_kv[e]`` is ``(group, slab)`` for run ``e`` of the order (None: no pages).
    ``states[i]`` is one fixed-size state; ``run_state[e]`` its index (or None).
    """

    kv_groups: List[PagedKVNeed] = field(default_factory=list)
    kv_slabs: List[int] = field(default_factory=list)
    run_kv: List[Optional[Tuple[int, int]]] = field(default_factory=list)
    states: List[StateNeed] = field(default_factory=list)
    run_state: List[Optional[int]] = field(default_factory=list)


_REGISTRY_OF_ROLE = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}


class _Layer:
    """The parts a ``LayerSpec`` names, built, and the block that arranges them.  The block kind is given the parts
    as keyword arguments under the spec's names and says by its constructor which it takes."""

    def __init__(self, spec, env):
        self.named = {name: _REGISTRY_OF_ROLE[ps.role].get(ps.kind)(ps.params, env) for name, ps in spec.parts.items()}
        block_cls = BLOCKS.get(spec.block)
        try:
            self.block = block_cls(**self.named)
        except TypeError as exc:
            raise ValueError(f"a {spec.block!r} block does not take the parts {sorted(self.named)}: {exc}") from None
        self.mixer = next((self.named[name] for name, ps in spec.parts.items() if ps.role == "mixer"), None)
        self.parts = [(self.named[name], ps) for name, ps in spec.parts.items()]


class DecoderModel:
    def __init__(self, plan: ModelPlan, env: BuildEnv):
        self.plan = plan
        self.env = env
        self.hidden_size = plan.hidden_size
        self.vocab_size = plan.vocab_size
        self.embedding = EMBEDDINGS.get(plan.embedding.kind)(plan.embedding.params, env)
        self.layers = [_Layer(spec, env) for spec in plan.layers]
        self.final_norm = NORMS.get(plan.final_norm.kind)(plan.final_norm.params, env)
        self.head = HEADS.get(plan.head.kind)(plan.head.params, env)
        if plan.head.params.get("tied"):
            if not hasattr(self.head, "share_embedding"):
                raise ValueError(f"the plan ties a {plan.head.kind!r} head to the embedding, but that head cannot share one")
            self.head.share_embedding(self.embedding)
        self.order = plan.run_order()
        self._parts = [(self.embedding, plan.embedding)]
        for layer in self.layers:
            self._parts.extend(layer.parts)
        self._parts += [(self.final_norm, plan.final_norm), (self.head, plan.head)]
        self._layout = self._make_cache_layout()

    # -- weights -----------------------------------------------------------
    def expected_tensors(self) -> Dict[str, TensorSpec]:
        """Checkpoint name -> shape and role, over all parts."""
        expected: Dict[str, TensorSpec] = {}
        for part, spec in self._parts:
            for local, tspec in part.weight_specs().items():
                if local not in spec.weights:
                    raise KeyError(f"plan gives no checkpoint name for tensor {local!r} of a {spec.kind!r} part")
                name = spec.weights[local]
                if name in expected and expected[name] != tspec:
                    raise ValueError(f"tensor {name} is wanted with two shapes: {expected[name]} and {tspec}")
                expected[name] = tspec
        return expected

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Hands every part its tensors (already checked, placed and typed by the loader)."""
        for part, spec in self._parts:
            part.bind({local: tensors[spec.weights[local]] for local in part.weight_specs()})
        for layer in self.layers:
            if getattr(layer.block, "plain_forms", None) is not None:
                layer.block.plain_forms = None     # what kernels kept of the parts pointed into the old tensors

    # -- caches ------------------------------------------------------------
    def _make_cache_layout(self) -> CacheLayout:
        layout = CacheLayout()
        latest_run_of_layer: Dict[int, int] = {}
        for e, li in enumerate(self.order):
            mixer = self.layers[li].mixer       # None: a layer without a mixer owns neither pages nor state
            need = mixer.cache_need() if mixer is not None else None
            source = getattr(mixer, "kv_from_layer", None)
            if need is None:
                layout.run_kv.append(None)
            elif source is not None:
                if source not in latest_run_of_layer:
                    raise ValueError(f"run {e} (layer {li}) reads the cache of layer {source}, which has not run before it")
                src = layout.run_kv[latest_run_of_layer[source]]
                if src is None or layout.kv_groups[src[0]] != need:
                    raise ValueError(f"layer {li} cannot read the cache of layer {source}: their cache needs differ")
                layout.run_kv.append(src)
            else:
                if need not in layout.kv_groups:
                    layout.kv_groups.append(need)
                    layout.kv_slabs.append(0)
                g = layout.kv_groups.index(need)
                layout.run_kv.append((g, layout.kv_slabs[g]))
                layout.kv_slabs[g] += 1
            sneed = mixer.state_need() if mixer is not None else None
            if sneed is None:
                layout.run_state.append(None)
            else:
                layout.run_state.append(len(layout.states))
                layout.states.append(sneed)
            latest_run_of_layer[li] = e
        return layout

    def cache_layout(self) -> CacheLayout:
        return self._layout

    # -- forward -----------------------------------------------------------
    def forward(self, ctx: StepContext, caches: List[LayerCache]) -> Optional[torch.Tensor]:
        """Runs the step's tokens; returns float32 logits ``[n_logit_rows, vocab]`` (None if none wanted)."""
        stream = ResidualStream(self.embedding.forward(ctx))
        for e, li in enumerate(self.order):
            self.layers[li].block.forward(stream, ctx, caches[e])
        if ctx.n_logit_rows == 0:
            return None
        h = self.final_norm.forward(stream, rows=ctx.logit_rows)
        return self.head.forward(h)
