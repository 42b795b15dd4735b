"""Decode-only steps replayed from captured HIP graphs.

A step in which every scheduled request computes exactly one token has a fixed shape once the
batch is padded to a bucket size: the same kernels on the same buffers, only the integers in the
metadata buffer change.  Such a step is captured once per bucket (model step + sampling) and
replayed afterwards, which removes a few hundred launches' worth of host time per step (the
reference launches every kernel of every step from the host, src/model/llama.cpp:104-129).

Padding rows have context length 0 and slot -1: they write no key, attend to nothing, and their
sampled ids are dropped.  Nothing inside a graph clears memory or allocates.

A captured launch must fit every step that replays it, so kernels that size their grid by the
context are captured for a bound on it.  There is one graph per (bucket, context class): a step
replays the graph of the smallest class that holds its longest context, so that an engine that
allows long sequences still runs short ones with the launches made for short ones.
"""
import contextlib
import gc
from typing import Dict, List

import numpy as np
import torch

from .runner import StepContext


@contextlib.contextmanager
def _no_collection():
    """No garbage collection while a stream is being captured: a collection that happens to start
    there may destroy device objects of an engine that is no longer used (its graphs, their memory
    pools), and releasing device memory during a capture ends the process."""
    was_enabled = gc.isenabled()
    gc.disable()   # (torch.cuda.graph collects once itself before the capture begins)
    try:
        yield
    finally:
        if was_enabled:
            gc.enable()

_BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256, 384, 512)
_CONTEXT_CLASSES = (1024, 2048, 8192, 32768)       # and the longest context the engine allows


class DecodeGraphs:
    def __init__(self, engine):
        self.engine = engine
        self.runner = engine.runner
        self.core = engine.core
        self.sampler = engine.sampler
        lim = self.runner.limits
        self.buckets = [b for b in _BUCKETS if b <= min(lim.max_seqs, lim.max_logit_rows, lim.max_tokens)]
        self.table_stride = lim.max_blocks_per_seq
        self.block_size = engine.config.block_size
        self.context_classes = [c for c in _CONTEXT_CLASSES if c < lim.max_context_len] + [lim.max_context_len]
        self.graphs: Dict[tuple, torch.cuda.CUDAGraph] = {}      # (bucket, context class) -> graph
        self._views = {}      # bucket -> (device view, pinned view, ints) of the metadata a replay uploads
        self.enabled = bool(self.buckets)

    def fits(self, n: int) -> bool:
        """May a decode-shaped step of n sequences be replayed from a graph?"""
        return self.enabled and 0 < n <= self.buckets[-1]

    def usable(self, plan) -> bool:
        return self.fits(len(plan)) and all(p.count == 1 and p.samples for p in plan)

    def _bucket(self, n: int) -> int:
        for b in self.buckets:
            if n <= b:
                return b
        raise RuntimeError("no bucket")

    def _context_class(self, context: int) -> int:
        for c in self.context_classes:
            if context <= c:
                return c
        raise RuntimeError(f"a context of {context} tokens exceeds what the engine allows")

    def _forward(self, layout, bucket, bound):
        """Only kernels of this package inside a graph: a library product may record nodes that
        clear memory, which do not replay reliably."""
        ops = self.runner.ops
        keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
        try:
            self._forward_inner(layout, bucket, bound)
        finally:
            ops.LIBRARY_GEMM_MIN_ROWS = keep

    def _forward_inner(self, layout, bucket, bound):
        step = StepContext(self.runner, layout)
        step.max_context_bound = bound
        logits = self.runner.model.forward(step)
        # the sampling parameters lie in the metadata buffer (padding rows: temperature 0, dropped)
        t, seeds, ids, idx = step.sampling_params()
        self.runner.ops.sample(logits, self.sampler.out[:bucket], t, seeds, ids, idx)

    def run(self, n: int) -> np.ndarray:
        """Runs the scheduler's current plan (n decode-shaped entries); returns the n sampled ids."""
        bucket = self._bucket(n)
        runner, s = self.runner, self.sampler
        # the class also fixes how many page ids per sequence a replay uploads and reads
        bound = self._context_class(max(self.core.plan_max_context, 1))
        stride = min(self.table_stride, -(-bound // self.block_size))
        layout = self.core.build_batch_from_plan(runner.host_buffer(), pad_rows=bucket, pad_seqs=bucket,
                                                 pad_logit_rows=bucket, table_stride=stride)
        assert layout.max_context <= bound
        runner._check(layout)
        views = self._views.get(bucket)
        if views is None or views[2] != layout.total:
            views = self._views[bucket] = (runner.meta_dev[:layout.total], runner._pinned[:layout.total], layout.total)
        views[0].copy_(views[1], non_blocking=True)
        # no event: the synchronous download below ends after this upload, so the pinned buffer
        # is free again when the next step fills it
        runner._upload_pending = False
        graph = self.graphs.get((bucket, bound))
        if graph is None:
            # eager once: creates every work buffer, and its result is this step's result (a capture
            # runs nothing, so the sampled ids stay where the eager pass left them)
            self._forward(layout, bucket, bound)
            torch.cuda.current_stream().synchronize()
            graph = torch.cuda.CUDAGraph()
            with _no_collection(), torch.cuda.graph(graph):
                self._forward(layout, bucket, bound)
            self.graphs[(bucket, bound)] = graph
            return s.download(n)
        graph.replay()
        return s.download(n)
