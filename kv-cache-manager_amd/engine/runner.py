"""The step function: one batch of (request, its next tokens) in, logits at the wanted places out.

``ModelRunner`` owns the model, the device side of the cache, the work buffers and the packed
metadata buffers.  ``execute`` runs exactly the rows it is given, prompt portions beside single
decoded tokens, from what earlier steps left in the cache.  The reference's step is
LlamaModel::forward (src/model/llama.cpp:54-141): one packed upload of integers, the layer loop,
the head on the wanted rows only.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from ..cache.manager import BatchLayout, CacheGroupSpec, HostCore
from ..cache.storage import KVStorage, StateStorage, bytes_per_block
from ..parts.base import BuildContext, KVCacheNeed, StateNeed, StepView
from ..parts.model import Model


@dataclass
class ModelLimits:
    """Largest step the work buffers are made for (src/model/llama.h:35-41, engine.cpp:38-45)."""
    max_tokens: int
    max_seqs: int
    max_logit_rows: int
    max_blocks_per_seq: int
    max_context_len: int


class Workspace:
    """Named device buffers with fixed capacity, reused by every step (stable addresses)."""

    def __init__(self, device, default_dtype, limits: ModelLimits, ops=None):
        self.device, self.default_dtype, self.limits, self.ops = device, default_dtype, limits, ops
        self.buffers: Dict[str, torch.Tensor] = {}
        self.row_caps = {"head_in": limits.max_logit_rows, "logits": limits.max_logit_rows}
        self.retired: List[torch.Tensor] = []

    def get(self, name, shape, dtype=None):
        dtype = dtype or self.default_dtype
        rows, cols = shape
        cap = self.row_caps.get(name, self.limits.max_tokens)
        if rows > cap:
            raise RuntimeError(f"step: batch exceeds model limits ({name}: {rows} rows > {cap})")
        key = (name, cols, dtype)
        buf = self.buffers.get(key)
        if buf is None:
            buf = torch.empty(cap, cols, dtype=dtype, device=self.device)
            self.buffers[key] = buf
        return buf[:rows]

    def scratch(self, name, rows, n, k):
        """Float32 scratch for the partial sums of a split-K product [rows, k] x [n, k], or None
        when that shape is not split.  Sized once for the most rows the split kernel takes."""
        key = ("scratch", name, n, k)
        if key not in self.buffers:
            # the number of splits changes with the rows: room for the worst row count
            need = 0
            if self.ops is not None:
                for m in range(1, min(512, self.limits.max_tokens) + 1):
                    splits = self.ops.skinny_splits(m, n, k)
                    if splits > 1:
                        need = max(need, splits * m * n)
            self.buffers[key] = torch.empty(need, dtype=torch.float32, device=self.device) if need else None
        return self.buffers[key]

    def flat(self, name, numel, dtype=torch.float32):
        """A flat buffer of at least ``numel`` elements.  Asked for more than it holds it is replaced
        by one at least half as large again; the old one is kept, not freed: recorded steps (graphs,
        launch lists) hold its address."""
        key = ("flat", name, dtype)
        buf = self.buffers.get(key)
        if buf is None or buf.numel() < numel:
            if buf is not None:
                self.retired.append(buf)
                numel = max(numel, buf.numel() + buf.numel() // 2)
            buf = torch.empty(numel, dtype=dtype, device=self.device)
            self.buffers[key] = buf
        return buf

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in list(self.buffers.values()) + self.retired if b is not None)


class StepContext(StepView):
    """What the parts see of one step (parts.base.StepView): where each array of the packed
    metadata lies on the device and on the host, and the work buffers."""

    def __init__(self, runner, layout: BatchLayout):
        self.runner, self.layout = runner, layout
        self.limits, self.attention_mode = runner.limits, runner.attn
        self.fold_norms, self.fold_rows, self.tune_products = runner.fold_norms, runner.fold_rows, runner.tune_products
        self.recording = False
        L = layout
        self.rows, self.real_rows = L.rows_padded, L.rows
        self.seqs, self.real_seqs = L.seqs_padded, L.seqs
        self.logit_rows_padded, self.logit_rows = L.logit_rows_padded, L.logit_rows
        self.max_context, self.max_run = L.max_context, L.max_run
        # what kernels that size their launch by the context may assume; a captured graph sets it
        # to the largest context the engine allows, so that the launch fits every replay
        self.max_context_bound = max(L.max_context, 1)
        self._leading = None
        d, h = runner.meta_dev, runner.meta_host
        T, S, R = self.rows, self.seqs, self.logit_rows_padded
        self.tokens = d[L.tokens:L.tokens + T]
        self.positions = d[L.positions:L.positions + T]
        self.ctx_lens = d[L.context_lens:L.context_lens + T]
        self.row_seq = d[L.row_seq:L.row_seq + T]
        self.run_start = d[L.run_start:L.run_start + S + 1]
        self.seq_start = d[L.seq_start:L.seq_start + S]
        self.seq_end = d[L.seq_end:L.seq_end + S]
        self.logit_row_index = d[L.logit_row_index:L.logit_row_index + R]
        self.state_slots = d[L.state_slots:L.state_slots + S]
        # the same arrays on the host, for parts that loop over sequences in Python
        self.host_positions = h[L.positions:L.positions + T]
        self.host_run_start = h[L.run_start:L.run_start + S + 1]
        self.host_seq_start = h[L.seq_start:L.seq_start + S]
        self.host_seq_end = h[L.seq_end:L.seq_end + S]
        self.host_state_slots = h[L.state_slots:L.state_slots + S]

    def leading_single_runs(self):
        """How many of the step's first sequences run exactly one token (the scheduler puts the
        decoding requests first); their rows are the step's first rows."""
        if self._leading is None:
            rs = self.host_run_start[:self.real_seqs + 1]
            n = 0
            while n < self.real_seqs and rs[n + 1] - rs[n] == 1:
                n += 1
            self._leading = n
        return self._leading

    def sampling_params(self):
        """(temperature f32, seeds i64 bit patterns, request ids i64, token index i32), one entry per
        padded logit row, on the device: they travel in the step's metadata buffer."""
        d, o, R = self.runner.meta_dev, self.layout.sampling, self.logit_rows_padded
        return (d[o:o + R].view(torch.float32), d[o + 2 * R:o + 4 * R].view(torch.int64),
                d[o + 4 * R:o + 6 * R].view(torch.int64), d[o + R:o + 2 * R])

    def slots(self, g):
        L = self.layout
        return self.runner.meta_dev[L.slots[g]:L.slots[g] + self.rows]

    def tables(self, g):
        L = self.layout
        return self.runner.meta_dev[L.tables[g]:L.tables[g] + self.seqs * L.table_stride[g]]

    def table_stride(self, g):
        return self.layout.table_stride[g]

    def ws(self, name, shape, dtype=None):
        return self.runner.workspace.get(name, shape, dtype)

    def scratch(self, name, rows, n, k):
        if rows > 512 or self.runner.dtype != torch.bfloat16:
            return None
        return self.runner.workspace.scratch(name, rows, n, k)

    def flat(self, name, numel, dtype=torch.float32):
        return self.runner.workspace.flat(name, numel, dtype)


class ModelRunner:
    def __init__(self, model: Model, core: HostCore, storages, limits: ModelLimits, dtype, device, attn="auto",
                 fold_norms=True, tune_products="off"):
        self.model, self.core, self.storages, self.limits = model, core, storages, limits
        self.dtype, self.device, self.attn = dtype, device, attn
        self.fold_norms, self.tune_products = bool(fold_norms), tune_products
        self.ops = model.ctx.ops
        self.fold_rows = self._fold_rows()
        self.workspace = Workspace(device, dtype, limits, self.ops)
        G = core.num_groups
        # (logits of every row may be asked for and fetched in portions: room for that many indices)
        ints = (4 * limits.max_tokens + 4 * limits.max_seqs + 1 + 7 * max(limits.max_logit_rows, limits.max_tokens)
                + G * (limits.max_tokens + limits.max_seqs * limits.max_blocks_per_seq) + 64)
        self._pinned = torch.empty(ints, dtype=torch.int32, pin_memory=True)
        self.meta_host = self._pinned.numpy()
        self.meta_dev = torch.zeros(ints, dtype=torch.int32, device=device)
        self.vocab_size = model.spec.vocab_size
        self._upload_done = torch.cuda.Event()
        self._upload_pending = False
        model.attach_caches(storages)

    # Every workgroup of a folded product reads all of the step's rows from L2 (rows x K per 8 or 16 output
    # columns), so a folded step's time grows with its rows by about a ninth of the layers' weight bytes at
    # L2 speed, while the unfolded path (rows shared through LDS, two norm launches a layer more) costs the
    # same from 1 to 16 rows.  Measured: at TinyLlama sizes (88 MB a layer) folding wins at every row count up
    # to 8 (batch 8: 1.00 against 1.13 ms), at Llama-3-8B sizes (436 MB a layer) up to 2 rows (3.61 against 3.89 ms; a tie
    # at 4 rows, 3.92 both ways; batch 8: 4.61 against 3.96 when it still folded), at Llama-2-7B sizes (405 MB) the same
    # (2 rows: 3.47 against 3.57 ms, 4 rows 3.71 both ways).  Rows x bytes of a layer's weights up to this pay.
    FOLD_ROWS_TIMES_LAYER_BYTES = 1.0e9

    @classmethod
    def fold_rows_for(cls, layer_bytes: float, most_rows: int) -> int:
        """The most rows a step may have for its norms to be folded, for layers of ``layer_bytes`` of weights."""
        return max(1, min(int(most_rows), int(cls.FOLD_ROWS_TIMES_LAYER_BYTES // max(1.0, float(layer_bytes)))))

    def _fold_rows(self) -> int:
        layers = max(1, len(self.model.spec.schedule))
        return self.fold_rows_for(self.model.step_bytes(1, 0) / layers, self.ops.FUSED_NORM_MAX_ROWS)

    def host_buffer(self) -> np.ndarray:
        """The pinned metadata buffer, once the previous step's upload no longer reads it."""
        if self._upload_pending:
            self._upload_done.synchronize()
            self._upload_pending = False
        return self.meta_host

    # ------------------------------------------------------------------------------ steps
    def _check(self, layout: BatchLayout, logits_in_portions=False):
        lim = self.limits
        if (layout.rows_padded > lim.max_tokens or layout.seqs_padded > lim.max_seqs
                or (layout.logit_rows_padded > lim.max_logit_rows and not logits_in_portions)
                or layout.max_context > lim.max_context_len
                or max(layout.table_stride + [0]) > lim.max_blocks_per_seq):
            raise RuntimeError(
                f"step: batch exceeds model limits (rows {layout.rows_padded}/{lim.max_tokens}, sequences "
                f"{layout.seqs_padded}/{lim.max_seqs}, logit rows {layout.logit_rows_padded}/{lim.max_logit_rows}, "
                f"context {layout.max_context}/{lim.max_context_len})")
        toks = self.meta_host[layout.tokens:layout.tokens + layout.rows]
        if layout.rows and (toks.min() < 0 or toks.max() >= self.vocab_size):
            raise ValueError(f"step: token id outside the vocabulary of {self.vocab_size}")

    def upload(self, layout: BatchLayout):
        """The one host-to-device copy of a step: its packed metadata."""
        n = layout.total
        self.meta_dev[:n].copy_(self._pinned[:n], non_blocking=True)
        self._upload_done.record()
        self._upload_pending = True

    def _begin(self, layout: BatchLayout, logits_in_portions=False) -> StepContext:
        self._check(layout, logits_in_portions)
        self.upload(layout)
        return StepContext(self, layout)

    def execute(self, layout: BatchLayout) -> Optional[torch.Tensor]:
        """Runs the batch whose metadata build_batch left in the host buffer.  Returns the logits
        [layout.logit_rows, vocab] (a view of a work buffer, valid until the next step), or None
        when no logits were asked for (the rows still run: their keys must reach the cache)."""
        if layout.rows == 0:
            return None
        if layout.logit_rows_padded > self.limits.max_logit_rows:
            raise RuntimeError(f"step: {layout.logit_rows_padded} logit rows exceed the limit of "
                               f"{self.limits.max_logit_rows} (use execute_to_host)")
        step = self._begin(layout)
        x, pending = self.model.run_layers(step)
        if layout.logit_rows_padded == 0:
            return None
        self.last_step = step
        return self.model.head_logits(step, x, pending, step.logit_row_index)[:layout.logit_rows]

    def execute_to_host(self, layout: BatchLayout) -> Optional[np.ndarray]:
        """As ``execute``, for any number of wanted rows: the head runs over them in portions of
        at most max_logit_rows and the logits are gathered in host memory [logit_rows, vocab]."""
        if layout.rows == 0:
            return None
        step = self._begin(layout, logits_in_portions=True)
        x, pending = self.model.run_layers(step)
        R = layout.logit_rows
        if R == 0:
            torch.cuda.current_stream().synchronize()
            return None
        out = np.empty((R, self.vocab_size), dtype=np.float32)
        cap = self.limits.max_logit_rows
        for lo in range(0, R, cap):
            hi = min(R, lo + cap)
            logits = self.model.head_logits(step, x, pending, step.logit_row_index[lo:hi])
            out[lo:hi] = logits.cpu().numpy()
        return out

    # ------------------------------------------------------------------------------- cost
    def step_bytes(self, contexts, rows=None, logit_rows=None) -> int:
        """Bytes a step has to read, as the loaded model and the cache storages count them: every weight it
        uses once, and the cache of the live requests (``contexts``: their lengths; one row and one wanted
        row per request unless said otherwise)."""
        n = len(contexts)
        weights = self.model.step_bytes(n if rows is None else rows, n if logit_rows is None else logit_rows)
        return weights + sum(s.bytes_read(c) for s in self.storages for c in contexts)

    def run_entries(self, entries, **pad) -> Optional[torch.Tensor]:
        """entries: (sequence id, start, count, want) as HostCore.build_batch takes them."""
        layout = self.core.build_batch(entries, self.host_buffer(), **pad)
        return self.execute(layout)


# --------------------------------------------------------------------------------- building
def plan_groups(model: Model, num_blocks: int, max_num_seqs: int) -> List[CacheGroupSpec]:
    groups = []
    for plan in model.groups:
        if isinstance(plan.need, KVCacheNeed):
            groups.append(CacheGroupSpec("window" if plan.need.window > 0 else "full", plan.need.window, num_blocks))
        else:
            groups.append(CacheGroupSpec("state", 0, 0))
    return groups


def make_storages(model: Model, num_blocks: int, block_size: int, max_num_seqs: int, dtype, device):
    out = []
    for g, plan in enumerate(model.groups):
        if isinstance(plan.need, KVCacheNeed):
            out.append(KVStorage(g, plan.need, len(plan.layers), num_blocks, block_size, dtype, device))
        else:
            out.append(StateStorage(g, plan.need, len(plan.layers), max_num_seqs, device))
    return out


def kv_bytes_per_block(model: Model, block_size: int, dtype) -> int:
    return sum(bytes_per_block(p.need, len(p.layers), block_size, dtype)
               for p in model.groups if isinstance(p.need, KVCacheNeed))
