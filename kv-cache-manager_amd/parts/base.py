"""What a part is: the interfaces the model assembly, the weight loader, the cache planner and
the step function rely on.  A part gets its sizes and constants as parameters and never learns
which model it is in.

Everything a part may rely on, and everything the engine asks of a part, is declared in this file:
``StepView`` (what ``step`` offers), the base classes with their optional capabilities as class
attributes (``capturable``, ``accepts_partial_sums``, ``rotates``, ``rotation_table``), and the
``Deferred`` convention for results that are not added up yet.  Nothing else is probed.
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
    """One layer: an arrangement (block kind) of named parts.  Every part that reports a cache need
    (``cache_need()``) owns a cache of its own, whatever its name and however many the layer has.
    ``cache_from`` makes parts read another part's cache instead: a string for every cache-using part
    of the layer (a layer's name: the part of the same name there; or ``layer.part``), or a dict from
    this layer's part names to such strings (parts it does not list keep their own)."""
    name: str
    block: str
    parts: Dict[str, PartSpec]
    cache_from: Optional[object] = None


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


# ------------------------------------------------------------------------------------- step
class StepView:
    """What a part sees of one step.  The engine's step context implements exactly this; a part
    uses nothing else of it.

    Shape of the step (host integers, fixed for a recorded step):
      rows, real_rows              rows the kernels run (padded) / rows that carry tokens
      seqs, real_seqs              sequences in the step (padded / real)
      logit_rows, logit_rows_padded
      max_run                      longest run of rows of one sequence (1: a decode-shaped step)
      max_context                  longest context among the rows
      max_context_bound            what launches sized by the context may assume (>= max_context; a
                                   recorded step sets it to the bound it was recorded for)
      limits                       the engine's ModelLimits (largest step the buffers are made for)
      attention_mode               "auto" | "v1" | "v2" (the engine option of that name)
      recording                    True while the step is being recorded for replay: a part may then
                                   call nothing but this package's kernels (ctx.ops) on device arrays
      fold_norms                   the engine option of that name: False keeps every norm a launch of its
                                   own, rounding exactly where the reference does
      fold_rows                    the most rows a step may have for its norms to be folded (the engine's
                                   estimate of where folding stops paying for this model's widths)
      tune_products                the engine option of that name ("off" | "heuristic" | "all"), handed to
                                   ops.gemm as ``tuning``

    Device arrays (int32, this step's metadata; all a capturable part may read):
      tokens[rows] positions[rows] ctx_lens[rows] row_seq[rows]
      run_start[seqs + 1] seq_start[seqs] seq_end[seqs] state_slots[seqs] logit_row_index[R]
      slots(g)[rows]               where each row's key and value go in group g (-1: nowhere)
      tables(g), table_stride(g)   page tables of group g, [seqs, table_stride(g)]

    The same on the host (NumPy views, for parts that loop over sequences in Python; reading them
    makes a part not capturable):
      host_positions host_run_start host_seq_start host_seq_end host_state_slots
      leading_single_runs()        how many of the first sequences run exactly one row

    Work memory (stable addresses, reused by every step):
      ws(name, (rows, cols), dtype=None)   a named 2-d work buffer in the compute dtype (or dtype)
      flat(name, numel, dtype=float32)     a named flat buffer of at least numel elements
      scratch(name, rows, n, k)            32-bit scratch for the split-K sums of a [rows, k] x [n, k]
                                           product, or None where that product is not split
      shared                               a dict in which parts of one step leave what later parts of
                                           the same step may reuse (keyed by the part; see Rotary)

    The members below are the defaults of a step that offers the least (what a part run on its own
    in a test needs to override is ``rows``, the arrays it reads and ``ws``)."""

    recording = False
    attention_mode = "auto"
    fold_norms = True
    fold_rows = 8
    tune_products = None
    max_run = 1
    limits = None

    @property
    def shared(self):
        return self.__dict__.setdefault("_shared", {})

    def scratch(self, name, rows, n, k):
        return None

    def leading_single_runs(self):
        return 0


class Deferred:
    """Convention for a result that is not a plain tensor yet (ops.PartialSums: the un-added split-K
    sums of a product).  It has ``materialize() -> tensor``; ``as_tensor`` turns either into a
    tensor.  A consumer that can take the deferred form itself says so (``accepts_partial_sums``)."""

    def materialize(self):
        raise NotImplementedError


def as_tensor(value):
    return value.materialize() if hasattr(value, "materialize") else value


class Part:
    """Base of every part.  Subclasses read ``params``, declare tensors in ``param_specs`` and get
    them (already on the device, in the precision their role asks for) through ``bind``."""

    # True when ``forward`` (``apply``) is a fixed sequence of this package's kernel launches for
    # a fixed step shape: every per-step value is read from the step's device arrays inside
    # kernels, never from the host copies (``step.host_*``), nothing is allocated and no library
    # routine is called.  Steps of a model whose parts are all capturable are recorded once per
    # shape and replayed (HIP graphs for decode steps, native launch lists for the others); one
    # part that is not keeps the whole model on the direct path.  The default is the safe one.
    capturable = False

    def __init__(self, params: dict, prefix: str, ctx: BuildContext):
        self.params = dict(params)
        self.prefix = prefix
        self.ctx = ctx
        self.w: Dict[str, torch.Tensor] = {}

    def sub_parts(self) -> Sequence["Part"]:
        """Parts this part builds and drives itself (an attention's position encoding)."""
        return ()

    def param_specs(self) -> List[ParamSpec]:
        return []

    def ignorable_tensors(self) -> Sequence[str]:
        """Checkpoint names that may be present without being used (derived buffers)."""
        return ()

    def bind(self, tensors: Dict[str, torch.Tensor]):
        self.w = dict(tensors)

    # What a step costs, for rooflines: a measurement asks the model, and the model asks its parts.
    def bytes_read(self, rows: int) -> int:
        """Bytes of its tensors a step of ``rows`` rows has to read: every tensor once, unless the part
        knows better (a table of which only ``rows`` rows are touched, experts that no row was routed to)."""
        return sum(t.numel() * t.element_size() for t in self.w.values())

    def flops(self, rows: int, attended: int = 0) -> float:
        """Floating-point operations of a step of ``rows`` rows: two per row and matrix element, unless the
        part knows better.  ``attended``: (row, key) pairs the step's rows see in all, for parts that attend."""
        return 2.0 * rows * sum(t.numel() for t in self.w.values() if t.dim() == 2)

    # A part of a layer that keeps something per request between steps says what (a mixer usually does;
    # any part of a layer may, and a layer may have several).
    def cache_need(self):
        """KVCacheNeed, StateNeed or None."""
        return None

    def attach_cache(self, storage, index: int, owner: bool = True):
        """storage: the group's device storage; index: this part's place in it; owner False: the
        cache belongs to another part and is only read."""
        self.cache, self.cache_index, self.cache_owner = storage, index, owner


class Norm(Part):
    # True: ``add`` may be a Deferred (un-added split-K sums, a product that has not run yet), which
    # the norm adds up or runs itself; False: the caller hands over a tensor (``as_tensor``).
    accepts_partial_sums = False
    # True: ``forward`` takes ``defer=True`` and may then return, instead of ``out``, a Deferred whose
    # scale is still to be applied by the product that consumes it (ops.NormedRows); the arrangement
    # asks for it only when the consuming part ``accepts_normed_rows``.
    defers = False

    def forward(self, x, out, add=None, rows=None):
        """out = norm(x (+ add)); when ``add`` is given and ``rows`` is not, x += add as well.
        x is the 32-bit residual stream; rows gathers source rows.  Returns the normed rows (``out``)."""
        raise NotImplementedError


class PositionEncoding(Part):
    # True: ``apply`` takes ``source=`` (the projection's un-added split-K sums) instead of
    # finished rows.
    accepts_partial_sums = False
    # False: q and k are left as they are (no encoding at this place), which lets an attention
    # kernel that stores k and v itself run without one.
    rotates = True

    def rotation_table(self, step, head_dim):
        """For encodings that rotate pairs (j, j + head_dim/2) by an angle that depends on the row
        alone: (cos, sin) of every row's angles, float32 [rows, head_dim/2, 2] on the device, for
        attention kernels that rotate inside.  None: this encoding is no such rotation (the
        attention then calls ``apply``)."""
        return None

    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
        """Transforms the q and k heads of the fused rows in place, given step.positions.  When a
        cache (k, v tensors) and slots are passed, also stores k (transformed) and v there and
        returns True; returning False leaves the store to the caller."""
        raise NotImplementedError


class Mixer(Part):
    # True: ``h`` may be a Deferred (ops.NormedRows) that the mixer's first product consumes as it is.
    accepts_normed_rows = False

    def forward(self, step, h):
        """h: normed hidden states [rows, H] in the compute dtype -> the mixer's output [rows, H]."""
        raise NotImplementedError


class FeedForward(Part):
    accepts_normed_rows = False      # as Mixer.accepts_normed_rows

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
    a tensor, a Deferred or None); it returns its own not-yet-added output, so that the addition
    fuses into the next norm.

    ``part_registries`` maps the names a LayerSpec may give this arrangement's parts to the
    registry each is looked up in (a registry object, or its name: "mixer", "feed_forward",
    "norm", "position").  Names it does not list fall back to the common ones: ``mixer``, ``ffn``
    and anything starting with ``norm``."""

    part_registries: Dict[str, object] = {}
    capturable = False      # as Part.capturable, for what the arrangement itself does between parts

    def __init__(self, parts: Dict[str, Part]):
        self.parts = parts

    def forward(self, step, x, pending):
        raise NotImplementedError
