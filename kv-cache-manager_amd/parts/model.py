"""Puts a model together from its description (ModelSpec): builds every part through the
registries, collects what the weight loader and the cache planner need to know, and runs the
layers in the order the description's schedule gives."""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Registry
from .base import BuildContext, KVCacheNeed, ModelSpec, Part, StateNeed, as_tensor

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
    layers: List[Tuple[str, str]]   # (layer name, part name) of every cache owner in this group, in order


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

    # --------------------------------------------------------------------------------- cost
    def _layer_parts_with_their_own(self) -> List[Part]:
        out, todo = [], [p for parts in self.layer_parts for p in parts.values()]
        while todo:
            p = todo.pop()
            out.append(p)
            todo.extend(p.sub_parts())
        return out

    def step_bytes(self, rows: int, logit_rows: int) -> int:
        """Bytes of weights a step of ``rows`` rows with ``logit_rows`` wanted rows has to read: every
        part's own answer (Part.bytes_read), every tensor once however often the schedule runs a layer."""
        parts = self._layer_parts_with_their_own() + [self.final_norm]
        return (self.embedding.bytes_read(rows) + sum(p.bytes_read(rows) for p in parts)
                + self.head.bytes_read(logit_rows))

    def step_flops(self, rows: int, logit_rows: int, attended: int) -> float:
        """Floating-point operations of such a step (Part.flops); a layer the schedule runs twice counts twice."""
        total = self.head.flops(logit_rows)
        for i in self.spec.schedule:
            todo = list(self.layer_parts[i].values())
            while todo:
                p = todo.pop()
                total += p.flops(rows, attended)
                todo.extend(p.sub_parts())
        return total

    def finish_binding(self):
        """Called by the loader after every part got its tensors: shares tied tables."""
        if self.spec.head.params.get("tied"):
            self.head.bind({"table": self.embedding.w["table"]})

    # -------------------------------------------------------------------------------- cache
    @staticmethod
    def _cache_need_of(part):
        """What a part of a layer says it needs of the cache manager: anything with a ``cache_need``
        method may own a cache (a Mixer is the usual case), whatever name the layer gives it."""
        ask = getattr(part, "cache_need", None)
        return ask() if callable(ask) else None

    def _resolve_cache_source(self, layer, slot) -> Optional[Tuple[str, str]]:
        """The (layer name, part name) whose cache the part ``slot`` of ``layer`` reads instead of owning
        one, or None when it owns its own.  ``LayerSpec.cache_from`` is a string that holds for every
        cache-using part of the layer, or a dict from part names to such strings; a string is a layer's
        name (then the part of the same name there is meant) or ``layer.part``."""
        src = layer.cache_from
        if isinstance(src, dict):
            src = src.get(slot)
        if src is None:
            return None
        if src in self.layer_names:
            return (src, slot)
        head, _, tail = src.rpartition(".")
        if head in self.layer_names:
            return (head, tail)
        raise ValueError(f"layer {layer.name}: cache_from {src!r} names no layer (a layer's name, or layer.part)")

    def _plan_cache_groups(self) -> List[CacheGroupPlan]:
        groups: List[CacheGroupPlan] = []
        self._cache_of: Dict[Tuple[str, str], Tuple[int, int]] = {}    # owner (layer, part) -> (group, index)
        self._cache_source: Dict[Tuple[str, str], Tuple[str, str]] = {}  # reader (layer, part) -> owner (layer, part)
        for layer, parts in zip(self.spec.layers, self.layer_parts):
            if isinstance(layer.cache_from, dict):
                unknown = sorted(set(layer.cache_from) - set(parts))
                if unknown:
                    raise ValueError(f"layer {layer.name}: cache_from names parts the layer does not have: {unknown}")
            for slot, part in parts.items():
                need = self._cache_need_of(part)
                if need is None:
                    continue
                if not isinstance(need, (KVCacheNeed, StateNeed)):
                    raise TypeError(f"layer {layer.name}, part {slot}: cache_need() must give a KVCacheNeed or a StateNeed")
                source = self._resolve_cache_source(layer, slot)
                if source is not None:
                    self._cache_source[(layer.name, slot)] = source
                    continue
                key = (layer.name, slot)
                for g, plan in enumerate(groups):
                    if plan.need == need:
                        self._cache_of[key] = (g, len(plan.layers))
                        plan.layers.append(key)
                        break
                else:
                    self._cache_of[key] = (len(groups), 0)
                    groups.append(CacheGroupPlan(need, [key]))
        for reader, owner in self._cache_source.items():
            if owner not in self._cache_of:
                raise ValueError(f"layer {reader[0]}, part {reader[1]} reads the cache of {owner[0]}.{owner[1]}, which owns none")
        return groups

    def attach_caches(self, storages):
        """storages[g]: device storage of group g (see cache.storage).  Every part that reported a
        cache need gets its place (or its owner's, read-only)."""
        for layer, parts in zip(self.spec.layers, self.layer_parts):
            for slot, part in parts.items():
                key = (layer.name, slot)
                owner = self._cache_source.get(key, key)
                if owner not in self._cache_of:
                    if self._cache_need_of(part) is not None:
                        raise RuntimeError(f"layer {layer.name}, part {slot} needs a cache that was not planned")
                    continue
                g, idx = self._cache_of[owner]
                part.attach_cache(storages[g], idx, owner=owner == key)

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
