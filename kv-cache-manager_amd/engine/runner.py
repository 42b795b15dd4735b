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
from ..parts.base import BuildContext, KVCacheNeed, StateNeed
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
        """A flat buffer of at least ``numel`` elements (grows if a larger one is asked for)."""
        key = ("flat", name, dtype)
        buf = self.buffers.get(key)
        if buf is None or buf.numel() < numel:
            buf = torch.empty(numel, dtype=dtype, device=self.device)
            self.buffers[key] = buf
        return buf

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in self.buffers.values() if b is not None)


class StepContext:
    """What the parts see of one step: where each array of the packed metadata lies on the device
    and on the host, the work buffers, and the attention entry point."""

    def __init__(self, runner, layout: BatchLayout):
        self.runner, self.layout = runner, layout
        L = layout
        self.rows, self.real_rows = L.rows_padded, L.rows
        self.seqs, self.real_seqs = L.seqs_padded, L.seqs
        self.logit_rows_padded, self.logit_rows = L.logit_rows_padded, L.logit_rows
        self.max_context, self.max_run = L.max_context, L.max_run
        # what kernels that size their launch by the context may assume; a captured graph sets it
        # to the largest context the engine allows, so that the launch fits every replay
        self.max_context_bound = max(L.max_context, 1)
        self.shared = {}    # what parts of one step compute once and share (keyed by the part kind)
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

    def attention(self, q, out, kcache, vcache, g, nh, nkv, hd, scale, window=0):
        self.runner.attention(self, q, out, kcache, vcache, g, nh, nkv, hd, scale, window)

    def decode_attention_fused(self, projection, out, kcache, vcache, g, nh, nkv, hd, scale, window, cos_sin, slots):
        """Rotation by ``cos_sin``, page write at ``slots`` and attention in one launch, straight
        from the QKV projection's result; False when this step or shape has no such kernel (then
        the caller runs them one after the other: the same values up to rounding)."""
        return self.runner.decode_attention_fused(self, projection, out, kcache, vcache, g, nh, nkv, hd, scale, window,
                                                  cos_sin, slots)


class ModelRunner:
    def __init__(self, model: Model, core: HostCore, storages, limits: ModelLimits, dtype, device, attn="auto"):
        self.model, self.core, self.storages, self.limits = model, core, storages, limits
        self.dtype, self.device, self.attn = dtype, device, attn
        self.ops = model.ctx.ops
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

    def host_buffer(self) -> np.ndarray:
        """The pinned metadata buffer, once the previous step's upload no longer reads it."""
        if self._upload_pending:
            self._upload_done.synchronize()
            self._upload_pending = False
        return self.meta_host

    # ------------------------------------------------------------------------- attention
    # Rows up to which a step is treated as decode-shaped by the partitioned attention kernel.
    DECODE_ATTENTION_MAX_ROWS = 512

    # The one-launch decode kernel walks a row's context chunk by chunk inside one workgroup:
    # right when contexts are moderate or there are enough rows to fill the chip; a few rows with
    # very long contexts are better cut into partitions that run in parallel.
    def _decode_parts_scratch(self, rows, nh, nkv, hd, bound):
        """Scratch for the decode kernel when it cuts long contexts of few rows into parts; sized at
        once for the worst case (rows x parts <= 256 / kv heads + rows), so that a captured graph's
        pointer stays good."""
        need = self.ops.attention_decode_fused_scratch(rows, nh, nkv, hd, bound)
        if need == 0:
            return None
        most_rows = min(self.DECODE_ATTENTION_MAX_ROWS, self.limits.max_tokens)
        worst = nh * (256 // nkv + 1 + most_rows) * (hd + 2)
        return self.workspace.flat("decode_parts", max(need, worst))

    def decode_attention_fused(self, step, projection, out, kcache, vcache, g, nh, nkv, hd, scale, window, cos_sin, slots):
        """From the QKV projection to the attention output.  Decode-shaped steps: one launch (and a
        small merge when few rows have long contexts).  Mixed steps (the scheduler puts decoding
        requests first): the leading single-token runs take that launch too, the rows after them
        are rotated and stored, then attended by the tiled kernel; a single-token run there would
        otherwise cost a whole tile of its own."""
        ops = self.ops
        if (self.attn != "auto" or window != 0 or out.dtype != torch.bfloat16
                or not ops.attention_decode_fused_supported(nh, nkv, hd, out.dtype, kcache.shape[2])):
            return False
        if step.max_run == 1:
            if step.rows > self.DECODE_ATTENTION_MAX_ROWS:
                return False
            bound = step.max_context_bound
            ops.attention_decode_fused(projection, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                                       step.ctx_lens, nh, nkv, hd, scale, cos_sin=cos_sin, slots=slots, rows=step.rows,
                                       max_context=bound, scratch=self._decode_parts_scratch(step.rows, nh, nkv, hd, bound))
            return True
        D, T, S = step.leading_single_runs(), step.real_rows, step.real_seqs
        if (D == 0 or D > self.DECODE_ATTENTION_MAX_ROWS
                or not ops.attention_prefill_supported(nh, nkv, hd, out.dtype, kcache.shape[2])):
            return False
        if isinstance(projection, ops.PartialSums):
            # three consumers here (decode rows, rotation of the others, tiled attention): add the
            # split sums up once instead of handing every single-token run to the tiled kernel
            projection = projection.materialize()
        stride = step.table_stride(g)
        ops.attention_decode_fused(projection, out, kcache, vcache, step.tables(g), stride, step.row_seq, step.ctx_lens,
                                   nh, nkv, hd, scale, cos_sin=cos_sin, slots=slots, rows=D, max_context=step.max_context,
                                   scratch=self._decode_parts_scratch(D, nh, nkv, hd, step.max_context))
        if (cos_sin is not None or slots is not None) and T > D:
            ops.rope_cache(projection[D:T], nh, nkv, hd, cos_sin=cos_sin[D:T] if cos_sin is not None else None,
                           slots=slots[D:T] if slots is not None else None, kcache=kcache, vcache=vcache,
                           block_size=kcache.shape[2], rows=T - D)
        need = ops.attention_prefill_scratch(T, nh, hd, step.max_context, step.max_run, S - D)
        scratch = self.workspace.flat("prefill_partials", need) if need else None
        ops.attention_prefill(projection, out, kcache, vcache, step.tables(g)[D * stride:], stride, step.run_start[D:],
                              step.seq_start[D:], S - D, step.max_run, nh, nkv, hd, scale, rows=T,
                              max_context=step.max_context, scratch=scratch)
        return True

    def attention(self, step, q, out, kcache, vcache, g, nh, nkv, hd, scale, window):
        """attn = "v1": the generic kernel, one pass over the whole context per (row, head); "v2" and
        "auto": for bfloat16, decode-shaped steps take the kernel that cuts contexts into partitions
        and merges them, steps with runs of positions take the tiled kernel; "v2" insists on the
        partitioned kernel for decode steps, "auto" prefers the one-launch kernel above where it
        applies.  The 32-bit path always takes v1, whose result does not depend on the batch."""
        ops = self.ops
        partitioned = (self.attn != "v1" and window == 0 and step.max_run == 1
                       and step.rows <= self.DECODE_ATTENTION_MAX_ROWS
                       and ops.attention_decode_supported(nh, nkv, hd, q.dtype, kcache.shape[2]))
        if self.attn == "v2" and not partitioned and q.dtype == torch.bfloat16 and step.max_run == 1:
            raise RuntimeError(f"attn=v2: the partitioned kernel does not take heads={nh} kv_heads={nkv} "
                               f"head_dim={hd} window={window} rows={step.rows}")
        if partitioned:
            bound = step.max_context_bound
            need = ops.attention_decode_scratch(step.rows, nh, hd, bound)
            scratch = self.workspace.flat("attention_partials", max(need, ops.attention_decode_scratch(
                min(self.DECODE_ATTENTION_MAX_ROWS, self.limits.max_tokens), nh, hd, self.limits.max_context_len)))
            ops.attention_decode(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                                 step.ctx_lens, nh, nkv, hd, scale, bound, scratch, rows=step.rows)
            return
        if (self.attn != "v1" and window == 0 and step.max_run > 1
                and ops.attention_prefill_supported(nh, nkv, hd, q.dtype, kcache.shape[2])):
            # runs of consecutive positions: keys are read once per 64 query rows, on the matrix cores
            need = ops.attention_prefill_scratch(step.real_rows, nh, hd, step.max_context, step.max_run, step.real_seqs)
            scratch = self.workspace.flat("prefill_partials", need) if need else None
            ops.attention_prefill(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.run_start,
                                  step.seq_start, step.real_seqs, step.max_run, nh, nkv, hd, scale,
                                  rows=step.real_rows, max_context=step.max_context, scratch=scratch)
            return
        ops.attention(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                      step.ctx_lens, nh, nkv, hd, scale, window, rows=step.rows)

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

    def _begin(self, layout: BatchLayout, logits_in_portions=False) -> StepContext:
        self._check(layout, logits_in_portions)
        n = layout.total
        self.meta_dev[:n].copy_(self._pinned[:n], non_blocking=True)
        self._upload_done.record()
        self._upload_pending = True
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
