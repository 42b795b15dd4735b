"""Decode-only steps replayed from captured HIP graphs.

A step in which every scheduled request computes exactly one token has a fixed shape once the
batch is padded to a bucket size: the same kernels on the same buffers, only the integers in the
metadata buffer change.  Such a step is captured once per bucket (model step + sampling) and
replayed afterwards, which removes a few hundred launches' worth of host time per step (the
reference launches every kernel of every step from the host, src/model/llama.cpp:104-129).

Padding rows have context length 0 and slot -1: they write no key, attend to nothing, and their
sampled ids are dropped.  Nothing inside a graph clears memory or allocates.
"""
from typing import Dict, List

import numpy as np
import torch

from .runner import StepContext

_BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256, 384, 512)


class DecodeGraphs:
    def __init__(self, engine):
        self.engine = engine
        self.runner = engine.runner
        self.core = engine.core
        self.sampler = engine.sampler
        lim = self.runner.limits
        self.buckets = [b for b in _BUCKETS if b <= min(lim.max_seqs, lim.max_logit_rows, lim.max_tokens)]
        self.table_stride = lim.max_blocks_per_seq
        self.graphs: Dict[int, torch.cuda.CUDAGraph] = {}
        self.enabled = bool(self.buckets)

    def usable(self, plan) -> bool:
        if not self.enabled or not plan or len(plan) > self.buckets[-1]:
            return False
        return all(p.count == 1 and p.samples for p in plan)

    def _bucket(self, n: int) -> int:
        for b in self.buckets:
            if n <= b:
                return b
        raise RuntimeError("no bucket")

    def _forward(self, layout, bucket):
        """Only kernels of this package inside a graph: a library product may record nodes that
        clear memory, which do not replay reliably."""
        ops = self.runner.ops
        keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
        try:
            self._forward_inner(layout, bucket)
        finally:
            ops.LIBRARY_GEMM_MIN_ROWS = keep

    def _forward_inner(self, layout, bucket):
        step = StepContext(self.runner, layout)
        step.max_context_bound = self.runner.limits.max_context_len
        logits = self.runner.model.forward(step)
        s = self.sampler
        self.runner.ops.sample(logits, s.out[:bucket], s.temperature[:bucket], s.seeds[:bucket],
                               s.request_ids[:bucket], s.token_index[:bucket])

    def run(self, plan) -> np.ndarray:
        n = len(plan)
        bucket = self._bucket(n)
        runner, s = self.runner, self.sampler
        layout = self.core.build_batch_from_plan(runner.host_buffer(), pad_rows=bucket, pad_seqs=bucket,
                                                 pad_logit_rows=bucket, table_stride=self.table_stride)
        runner._check(layout)
        total = layout.total
        runner.meta_dev[:total].copy_(runner._pinned[:total], non_blocking=True)
        runner._upload_done.record()
        runner._upload_pending = True
        # sampling parameters for the real rows; padding rows keep temperature 0 (argmax, dropped)
        temps = np.zeros(bucket, dtype=np.float32)
        seeds = np.zeros(bucket, dtype=np.uint64)
        reqs = np.zeros(bucket, dtype=np.int64)
        idx = np.zeros(bucket, dtype=np.int32)
        for k, p in enumerate(plan):
            temps[k], seeds[k], reqs[k], idx[k] = p.temperature, p.seed & ((1 << 64) - 1), p.id, p.gen_index
        s.temperature[:bucket].copy_(torch.from_numpy(temps))
        s.seeds[:bucket].copy_(torch.from_numpy(seeds.view(np.int64)))
        s.request_ids[:bucket].copy_(torch.from_numpy(reqs))
        s.token_index[:bucket].copy_(torch.from_numpy(idx))

        graph = self.graphs.get(bucket)
        if graph is None:
            self._forward(layout, bucket)                 # eager once: creates every work buffer
            torch.cuda.current_stream().synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._forward(layout, bucket)
            self.graphs[bucket] = graph
        graph.replay()
        s._host[:bucket].copy_(s.out[:bucket])            # synchronous download
        return s._host[:n].numpy().copy()
