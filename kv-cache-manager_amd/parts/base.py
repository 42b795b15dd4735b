"""What a part is: the interfaces the model assembly, the weight loader, the cache planner and
the step function rely on.  A part gets its sizes and constants as parameters and never learns
which model it is in.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch


# ------------------------------------------------------------------------------- description
@dataclass(frozen=True)
class PartSpec:
    """One part as data: its registered kind, its parameters, and the prefix under which its
    tensors are stored in the checkpoint."""
    kind: str
    params: dict = field(default_factory=dict)
    prefix: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (block kind) of named parts.  ``cache_from`` names another layer
    whose cache this layer's mixer reads instead of owning one."""
    name: str
    block: str
    parts: Dict[str, PartSpec]
    cache_from: Optional[str] = None


@dataclass(frozen=True)
class ModelSpec:
    """A whole model as data.  ``schedule`` is the order in which layers run: indices into
    ``layers``; an index may appear more than once."""
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[int, ...]
    final_norm: PartSpec
    head: PartSpec
    max_position: int = 0


# ---------------------------------------------------------------------------------- weights
@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part wants.  ``sources`` are (checkpoint name, shape) pairs concatenated along
    dim 0 in that order (one pair = taken as it is).  ``role`` decides the stored precision:
      matrix / table  the compute dtype (bfloat16 when serving, float32 in the 32-bit path)
      vector          as stored when that is 32-bit, else the compute dtype
      index           integer tables, kept as int32."""
    name: str
    sources: Tuple[Tuple[str, Tuple[int, ...]], ...]
    role: str = "matrix"

    @property
    def shape(self):
        first = self.sources[0][1]
        return (sum(s[1][0] for s in self.sources),) + tuple(first[1:])


# ------------------------------------------------------------------------------------ cache
@dataclass(frozen=True)
class KVCacheNeed:
    """Paged keys and values: every key (window 0) or the last ``window`` of them."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size state per request: one slot of this shape and dtype per admitted request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


# ------------------------------------------------------------------------------------ build
@dataclass
class BuildContext:
    dtype: torch.dtype          # compute / storage dtype: torch.bfloat16 or torch.float32
    device: torch.device
    hidden_size: int
    block_size: int
    ops: object                 # the kernel module (kvcm_amd.ops)


class Part:
    """Base of every part.  Subclasses read ``params``, declare tensors in ``param_specs`` and get
    them (already on the device, in the precision their role asks for) through ``bind``."""

    def __init__(self, params: dict, prefix: str, ctx: BuildContext):
        self.params = dict(params)
        self.prefix = prefix
        self.ctx = ctx
        self.w: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> List[ParamSpec]:
        return []

    def ignorable_tensors(self) -> Sequence[str]:
        """Checkpoint names that may be present without being used (derived buffers)."""
        return ()

    def bind(self, tensors: Dict[str, torch.Tensor]):
        self.w = dict(tensors)


class Norm(Part):
    def forward(self, x, out, add=None, rows=None):
        """out = norm(x (+ add)); when ``add`` is given and ``rows`` is not, x += add as well.
        x is the 32-bit residual stream; rows gathers source rows."""
        raise NotImplementedError


class PositionEncoding(Part):
    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
        """Transforms the q and k heads of the fused rows in place, given step.positions.  When a
        cache (k, v tensors) and slots are passed, also stores k (transformed) and v there and
        returns True; returning False leaves the store to the caller."""
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        """KVCacheNeed, StateNeed or None."""
        return None

    def attach_cache(self, storage, index: int, owner: bool = True):
        """storage: the group's device storage; index: this layer's place in it; owner False: the
        cache belongs to another layer and is only read."""
        self.cache, self.cache_index, self.cache_owner = storage, index, owner

    def forward(self, step, h):
        """h: normed hidden states [rows, H] in the compute dtype -> the mixer's output [rows, H]."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, step, h):
        raise NotImplementedError


class Embedding(Part):
    def forward(self, step, out):
        raise NotImplementedError


class Head(Part):
    def forward(self, step, h, out):
        raise NotImplementedError


class Block:
    """An arrangement of parts.  ``forward`` takes the residual stream x (32-bit, updated in
    place) and the output of the previous block that has not been added to x yet (``pending``,
    may be None); it returns its own not-yet-added output, so that the addition fuses into the
    next norm."""

    def __init__(self, parts: Dict[str, Part]):
        self.parts = parts

    def forward(self, step, x, pending):
        raise NotImplementedError
