"""Recorded steps: the Python side of the native step loop (csrc/hip/native_engine.hip).

A step of a model whose parts are all capturable is a fixed list of kernel launches once its shape
is fixed: the same kernels on the same buffers, only the integers in the metadata buffer change.
The first step of a shape runs through the parts while every launch is recorded into a step program
(model step + sampling); later steps of that shape never reach Python's part code: the native engine
schedules, builds and uploads the metadata, replays the program, downloads the sampled ids and
updates the scheduler (the reference launches every kernel of every step from its C++ step function,
src/model/llama.cpp:104-129, inside Engine::step, src/engine/engine.cpp:73-90).

Shapes are canonical (see native_engine.hip): padding rows have context length 0 and slot -1, they
write no key, attend to nothing, and their sampled ids are dropped.  Decode-shaped steps (every
request computes one token) of up to GRAPH_ROWS rows are additionally captured into a HIP graph, one
per (batch bucket, context class): a launch must fit every step that replays it, so kernels that size
their grid by the context are recorded for a bound on it, and a step replays the graph of the smallest
class that holds its longest context.  Nothing inside a recorded step clears memory or allocates.
"""
import contextlib
import ctypes as C
import gc
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .runner import StepContext

# Decode-shaped steps of more rows replay their program without a graph, and with the library's
# products, which a graph may not hold: measured at TinyLlama sizes, graph with this package's products
# against program with the library's: 96 rows 1.94 / 2.14 ms, 128 rows 2.15 / 2.20, 192 rows 2.87 / 2.62,
# 256 rows 3.21 / 2.88 (beyond 128 rows this package's kernel streams the weights once per 128 rows).
GRAPH_ROWS = 128


@contextlib.contextmanager
def _no_collection():
    """No garbage collection while a stream is being captured: a collection that happens to start
    there may destroy device objects of an engine that is no longer used (its graphs, their memory
    pools), and releasing device memory during a capture ends the process."""
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if was_enabled:
            gc.enable()


@dataclass(frozen=True)
class StepShape:
    """The canonical shape a step is recorded and replayed in."""
    rows: int
    seqs: int
    leading: int            # single-token runs at the front (padded to a bucket)
    logit_rows: int
    max_run: int
    context_bound: int
    table_stride: int


class RecordedStepContext(StepContext):
    """The step as a recorded program may see it: every host integer is the shape's, not the
    batch's, so that the launches fit every step of the shape."""

    def __init__(self, runner, layout, shape: StepShape):
        super().__init__(runner, layout)
        assert (self.rows, self.seqs, self.logit_rows_padded) == (shape.rows, shape.seqs, shape.logit_rows)
        self.real_rows, self.real_seqs, self.logit_rows = shape.rows, shape.seqs, shape.logit_rows
        self.max_run = shape.max_run
        self.max_context = self.max_context_bound = shape.context_bound
        self._leading = shape.leading
        self.recording = True


class RecordedSteps:
    def __init__(self, engine, use_graphs=True):
        self.engine, self.runner, self.core, self.sampler = engine, engine.runner, engine.core, engine.sampler
        ops = self.ops = self.runner.ops
        self.lib = ops.lib()
        lim = self.runner.limits
        self.stream = torch.cuda.Stream()          # default priority; every step of this engine runs on it
        names = ("kvcm_sched_schedule_summary", "kvcm_build_batch_from_plan_shaped", "kvcm_sched_update_sampled",
                 "kvcm_last_error", "kvcm_sched_add", "kvcm_sched_idle", "kvcm_sched_collect_finished",
                 "kvcm_finished_get", "kvcm_finished_clear")
        fns = (C.c_uint64 * len(names))(*[self.core.native_function(n) for n in names])
        s = self.sampler
        self._h = self.lib.kvcm_engine_new(
            self.core.handle, fns, self.runner._pinned.data_ptr(), self.runner.meta_dev.data_ptr(), self.runner.meta_dev.numel(),
            s.out.data_ptr(), s._host.data_ptr(), s.max_rows, self.core.num_groups, engine.config.block_size,
            lim.max_context_len, lim.max_tokens, lim.max_seqs, lim.max_logit_rows, GRAPH_ROWS if use_graphs else 0,
            self.stream.cuda_stream)
        if not self._h:
            raise ops.KernelError(self.lib.kvcm_hip_last_error().decode())
        self._out = (C.c_int64 * 20)()
        self._info = (C.c_int64 * 8)()
        self.last_host_us = 0            # of the last replayed step: host time from scheduling to the last launch
        self.shape: Optional[StepShape] = None
        self.recorded_shapes = {}        # StepShape -> "graph" | "program"
        torch.cuda.synchronize()         # weights and caches were written on other streams

    def __del__(self):
        if getattr(self, "_h", None):
            self.lib.kvcm_engine_delete(self._h)
            self._h = None

    # ------------------------------------------------------------------------------- one step
    def plan(self, now: float, again=False):
        """Runs the scheduler.  -> (entries, prompt tokens, decoding sequences, sampling entries); sets
        ``shape`` (None when the plan fits no canonical shape), ``has_program`` and ``wants_graph``.
        ``again``: the scheduler is not run; the plan a native caller's kvcm_engine_step made and could
        not run (its shape has no program yet) is taken up."""
        o = self._out
        n = self.lib.kvcm_engine_last_plan(self._h, o) if again else self.lib.kvcm_engine_plan(self._h, float(now), o)
        if n < 0:
            raise self.ops.KernelError(self.lib.kvcm_hip_last_error().decode())
        self.core.plan_max_context, self.core.plan_rows, self.core.plan_leading, self.core.plan_max_run = o[5], o[6], o[7], o[8]
        self.shape = StepShape(*[int(o[k]) for k in range(11, 18)]) if o[10] else None
        self.has_program, self.wants_graph = bool(o[18]), bool(o[19])
        return n, int(o[1]), int(o[2]), int(o[3])

    def replay(self, now: float, defer_update=False):
        """The planned step from its program, natively, scheduler update included.  -> (rows, sequences,
        sampled ids) or None when the shape has no program yet.  ``defer_update``: the update is left
        to the caller, who gets the sampled ids (else the third value is None)."""
        rc = self.lib.kvcm_engine_run(self._h, float(now), int(defer_update), self._info)
        if rc < 0:
            raise self.ops.KernelError(self.lib.kvcm_hip_last_error().decode())
        if rc == 0:
            return None
        self.runner._upload_pending = False      # the native step waited for its stream
        self.last_host_us = int(self._info[4])
        ids = self.sampler._host[:int(self._info[2])].numpy().copy() if defer_update else None
        return int(self._info[0]), int(self._info[1]), ids

    def record(self, sampling: int):
        """Runs the planned step through the model's parts on this engine's stream, recording every
        launch, registers the program (captured as a graph where the shape wants one) and returns
        (layout, sampled ids): this pass's results are the step's results."""
        shape, runner, ops = self.shape, self.runner, self.ops
        with torch.cuda.stream(self.stream), _no_collection():
            layout = self.core.build_batch_from_plan(runner.host_buffer(), pad_rows=shape.rows, pad_seqs=shape.seqs,
                                                     pad_logit_rows=shape.logit_rows, table_stride=shape.table_stride,
                                                     pad_leading=shape.leading)
            assert layout.max_context <= shape.context_bound
            runner._check(layout)
            runner.upload(layout)
            step = RecordedStepContext(runner, layout, shape)
            program = ops.StepProgram()
            # only kernels of this package inside a graph: a library product may record nodes that
            # clear memory, which do not replay reliably
            keep = ops.LIBRARY_GEMM_MIN_ROWS
            if self.wants_graph:
                ops.LIBRARY_GEMM_MIN_ROWS = 0
            try:
                with ops.recording(program):
                    logits = runner.model.forward(step)
                    t, seeds, ids, idx = step.sampling_params()
                    ops.sample(logits, self.sampler.out[:shape.logit_rows], t, seeds, ids, idx)
            finally:
                ops.LIBRARY_GEMM_MIN_ROWS = keep
            sampled = self.sampler.download(sampling)
            if self.lib.kvcm_engine_register(self._h, program.release(), int(self.wants_graph)) != 0:
                raise ops.KernelError(self.lib.kvcm_hip_last_error().decode())
            self.recorded_shapes[shape] = "graph" if self.wants_graph else "program"
        return layout, sampled

    @property
    def native_handle(self):
        """The native engine object (csrc/hip/kvcm_hip.h: kvcm_engine_add / step / idle / take_finished):
        what a native caller holds to serve requests without the interpreter once the shapes it meets
        are recorded."""
        return self._h

    # ---------------------------------------------------------------------------------- info
    def stats(self) -> dict:
        out = (C.c_int64 * 4)()
        self.lib.kvcm_engine_stats(self._h, out)
        return dict(programs=int(out[0]), graphs=int(out[1]), steps_replayed=int(out[2]), steps_as_graph=int(out[3]))

    def graph_shapes(self):
        """(batch bucket, context class) of every captured decode graph."""
        return sorted((s.rows, s.context_bound) for s, kind in self.recorded_shapes.items() if kind == "graph")
