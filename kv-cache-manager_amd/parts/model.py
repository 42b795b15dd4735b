"""Puts a model together from its description (ModelSpec): builds every part through the
registries, collects what the weight loader and the cache planner need to know, and runs the
layers in the order the description's schedule gives."""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Registry
from .base import BuildContext, KVCacheNeed, Mixer, ModelSpec, Part, StateNeed, as_tensor

# registries by the names a block arrangement may use in ``part_registries``
_REGISTRY_NAMES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "ffn": FEED_FORWARDS, "norm": NORMS,
                   "position": POSITIONS}


def _registry_for(slot, block_class=None):
    """The registry a part named ``slot`` of a layer is built from: what the layer's block
    arrangement declares for that name (``Block.part_registries``), else the common names."""
    declared = getattr(block_class, "part_registries", None) or {}
    if slot in declared:
        reg = declared[slot]
        if isinstance(reg, Registry):
            return reg
        if reg in _REGISTRY_NAMES:
            return _REGISTRY_NAMES[reg]
        raise KeyError(f"{getattr(block_class, '__name__', block_class)}.part_registries[{slot!r}] names no registry: "
                       f"{reg!r} (a Registry, or one of {sorted(_REGISTRY_NAMES)})")
    if slot == "mixer":
        return MIXERS
    if slot == "ffn":
        return FEED_FORWARDS
    if slot.startswith("norm"):
        return NORMS
    raise KeyError(f"a block part named {slot!r} has no registry: the block arrangement must list it in "
                   f"part_registries (common names: mixer, ffn, norm*)")


@dataclass
class CacheGroupPlan:
    """Layers whose caches have the same shape and rule share one group (and one page table)."""
    need: object                 # KVCacheNeed or StateNeed
    layers: List[str]            # names of the layers that own a cache in this group, in order


class Model:
    def __init__(self, spec: ModelSpec, ctx: BuildContext):
        self.spec, self.ctx = spec, ctx
        self.embedding = EMBEDDINGS.get(spec.embedding.kind)(spec.embedding.params, spec.embedding.prefix, ctx)
        self.final_norm = NORMS.get(spec.final_norm.kind)(spec.final_norm.params, spec.final_norm.prefix, ctx)
        self.head = HEADS.get(spec.head.kind)(spec.head.params, spec.head.prefix, ctx)
        self.layer_names = [l.name for l in spec.layers]
        if len(set(self.layer_names)) != len(self.layer_names):
            raise ValueError("layer names must be unique")
        self.blocks = []
        self.layer_parts: List[Dict[str, Part]] = []
        for layer in spec.layers:
            block_class = BLOCKS.get(layer.block)
            parts = {slot: _registry_for(slot, block_class).get(ps.kind)(ps.params, ps.prefix, ctx)
                     for slot, ps in layer.parts.items()}
            self.layer_parts.append(parts)
            self.blocks.append(block_class(parts))
        for i in spec.schedule:
            if not 0 <= i < len(self.blocks):
                raise ValueError(f"schedule names layer {i}, the model has {len(self.blocks)}")
        self.groups = self._plan_cache_groups()

    # ------------------------------------------------------------------------------ weights
    def all_parts(self) -> List[Part]:
        out = [self.embedding]
        for parts in self.layer_parts:
            out.extend(parts.values())
        out += [self.final_norm, self.head]
        return out

    def every_part(self) -> List[Part]:
        """All parts, with the parts that parts drive themselves."""
        out, todo = [], list(self.all_parts())
        while todo:
            p = todo.pop()
            out.append(p)
            todo.extend(p.sub_parts())
        return out

    @property
    def capturable(self) -> bool:
        """May a step of this model be recorded once and replayed?  Only when every part and every
        block arrangement says so of itself."""
        return all(p.capturable for p in self.every_part()) and all(b.capturable for b in self.blocks)

    def not_capturable(self) -> List[str]:
        names = [type(p).__name__ for p in self.every_part() if not p.capturable]
        names += [type(b).__name__ for b in self.blocks if not b.capturable]
        return sorted(set(names))

    def finish_binding(self):
        """Called by the loader after every part got its tensors: shares tied tables."""
        if self.spec.head.params.get("tied"):
            self.head.bind({"table": self.embedding.w["table"]})

    # -------------------------------------------------------------------------------- cache
    def _plan_cache_groups(self) -> List[CacheGroupPlan]:
        groups: List[CacheGroupPlan] = []
        self._cache_of: Dict[str, Tuple[int, int]] = {}    # owner layer name -> (group, index)
        for layer, parts in zip(self.spec.layers, self.layer_parts):
            mixer = parts.get("mixer")
            if mixer is None or layer.cache_from is not None:
                continue
            need = mixer.cache_need()
            if need is None:
                continue
            if not isinstance(need, (KVCacheNeed, StateNeed)):
                raise TypeError(f"layer {layer.name}: cache_need() must give a KVCacheNeed or a StateNeed")
            for g, plan in enumerate(groups):
                if plan.need == need:
                    self._cache_of[layer.name] = (g, len(plan.layers))
                    plan.layers.append(layer.name)
                    break
            else:
                self._cache_of[layer.name] = (len(groups), 0)
                groups.append(CacheGroupPlan(need, [layer.name]))
        for layer in self.spec.layers:
            if layer.cache_from is not None and layer.cache_from not in self._cache_of:
                raise ValueError(f"layer {layer.name} reads the cache of {layer.cache_from!r}, which owns none")
        return groups

    def attach_caches(self, storages):
        """storages[g]: device storage of group g (see cache.storage)."""
        for layer, parts in zip(self.spec.layers, self.layer_parts):
            mixer = parts.get("mixer")
            if not isinstance(mixer, Mixer):
                continue
            owner_name = layer.cache_from or layer.name
            if owner_name not in self._cache_of:
                continue
            g, idx = self._cache_of[owner_name]
            mixer.attach_cache(storages[g], idx, owner=layer.cache_from is None)

    # --------------------------------------------------------------------------------- step
    def run_layers(self, step):
        """Embeds the step's rows and runs every scheduled layer.  Returns the residual stream and
        the last block's output that is not added to it yet."""
        x = step.ws("residual", (step.rows, self.spec.hidden_size), torch.float32)
        self.embedding.forward(step, x)
        pending = None
        for i in self.spec.schedule:
            pending = self.blocks[i].forward(step, x, pending)
        return x, pending

    def head_logits(self, step, x, pending, row_index: torch.Tensor, out: Optional[torch.Tensor] = None):
        """32-bit logits [len(row_index), vocab] of the given rows: final norm (with the pending
        addition) and output head on those rows only (src/model/llama.cpp:126-128)."""
        R = row_index.numel()
        h_last = step.ws("head_in", (R, self.spec.hidden_size))
        if not self.final_norm.accepts_partial_sums:
            pending = as_tensor(pending)
        self.final_norm.forward(x, h_last, add=pending, rows=row_index)
        logits = out if out is not None else step.ws("logits", (R, self.spec.vocab_size), torch.float32)
        return self.head.forward(step, h_last, logits)

    def forward(self, step, logits_out: Optional[torch.Tensor] = None):
        """Logits [step.logit_rows_padded, vocab] for the rows in step.logit_row_index."""
        x, pending = self.run_layers(step)
        return self.head_logits(step, x, pending, step.logit_row_index, logits_out)
