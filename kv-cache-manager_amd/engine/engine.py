"""The engine: scheduler + cache manager + model step + sampler behind the reference's API
(src/engine/engine.h:29-52): add / step / take_finished / idle / score, plus generate().

One step = schedule (native) -> packed batch metadata (native) -> one upload -> model step on
the GPU -> sample -> one download of the sampled ids -> update (native)
(src/engine/engine.cpp:73-90)."""
import time
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import Finished
from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler
from .build import build_runner


@dataclass
class StepInfo:
    rows: int = 0
    seqs: int = 0
    prefill_tokens: int = 0
    decode_seqs: int = 0
    ms: float = 0.0


class Engine:
    def __init__(self, model_dir: Optional[str] = None, config: Optional[EngineConfig] = None, *,
                 architecture=None, model_config=None, tensors=None, device="cuda:0"):
        self.config = config or EngineConfig()
        self.runner, self.core, self.model, self.model_config = build_runner(
            model_dir, self.config, architecture=architecture, model_config=model_config, tensors=tensors, device=device)
        self.sampler = Sampler(self.runner.ops, self.runner.device, self.runner.limits.max_logit_rows)
        self._next_id = 0
        self._score_id = -1
        # teacher forcing: live request id -> its given tokens (dropped when the request finishes);
        # request id -> [given tokens, vocab] logits kept for it until ``forced_logits`` hands them out
        self._forced, self._forced_logits = {}, {}
        self._t0 = time.perf_counter()
        self.config = self.runner.engine_config      # as built (max_seq_len within the model's range)
        # Recorded steps replay a fixed launch sequence: only for models whose parts all declare that
        # their launches depend on the step's shape alone (Part.capturable).  use_programs: steps are
        # recorded per shape and replayed natively; use_graphs: decode-shaped ones also as HIP graphs.
        self.recorded = None
        if (self.config.use_programs or self.config.use_graphs) and self.model.capturable:
            from .graphs import RecordedSteps
            self.recorded = RecordedSteps(self, use_graphs=self.config.use_graphs)

    @property
    def decode_graphs(self):
        """The recorded-steps executor when it captures decode graphs, else None."""
        return self.recorded if (self.recorded is not None and self.config.use_graphs) else None

    @property
    def programs(self):
        return self.recorded if (self.recorded is not None and self.config.use_programs) else None

    # ------------------------------------------------------------------------------ clock
    def now(self) -> float:
        return time.perf_counter() - self._t0

    def reset_clock(self):
        self._t0 = time.perf_counter()

    # --------------------------------------------------------------------------- requests
    def add_request(self, tokens: Sequence[int], max_new_tokens: int, temperature: float = 0.0, seed: int = 0,
                    request_id: Optional[int] = None, arrival: Optional[float] = None,
                    forced: Optional[Sequence[int]] = None) -> int:
        """``forced``: the tokens this request "generates", given instead of sampled (teacher forcing):
        the request runs through admission, portions, preemption and prefix hits like any other, every
        sampled id is replaced by the next forced token, and ``forced_logits`` returns what it was
        sampled from.  max_new_tokens is then len(forced)."""
        if request_id is None:
            request_id = self._next_id
        self._next_id = max(self._next_id, request_id + 1)
        toks = [int(t) for t in tokens]
        V = self.model.spec.vocab_size
        if not toks:
            raise ValueError("a request needs at least one token")
        if min(toks) < 0 or max(toks) >= V:
            raise ValueError(f"token id outside the vocabulary of {V}")
        if forced is not None:
            forced = [int(t) for t in forced]
            if not forced or min(forced) < 0 or max(forced) >= V:
                raise ValueError("forced tokens must be a non-empty list of ids inside the vocabulary")
            max_new_tokens = len(forced)
            self._forced[request_id] = forced
            self._forced_logits[request_id] = np.full((len(forced), V), np.nan, dtype=np.float32)
        self.core.sched_add(request_id, toks, int(max_new_tokens), float(temperature), int(seed),
                            self.now() if arrival is None else arrival)
        return request_id

    add = add_request

    def idle(self) -> bool:
        return self.core.idle()

    def take_finished(self) -> List[Finished]:
        done = self.core.take_finished()
        for f in done:
            self._forced.pop(f.id, None)       # nothing of a finished request stays behind but the logits it asked for
        return done

    # ------------------------------------------------------------------------------- step
    def step(self, planned_natively=False) -> StepInfo:
        """One step.  ``planned_natively``: a native caller's kvcm_engine_step has run the scheduler already
        and found no program for the plan's shape; the scheduler is not run again, the planned step runs
        through the parts and is recorded."""
        info = StepInfo()
        t_start = self.now()
        rec, forcing = self.recorded, bool(self._forced)
        if planned_natively and rec is None:
            raise RuntimeError("step(planned_natively=True) needs recorded steps (a capturable model, use_programs or use_graphs)")
        ids = None
        if rec is None:
            n, info.prefill_tokens, info.decode_seqs, sampling, _ = self.core.schedule_summary(t_start)
            if n:
                ids = self._step_direct(info, sampling)
        else:
            n, info.prefill_tokens, info.decode_seqs, sampling = rec.plan(t_start, again=planned_natively)
            if n:
                # (with use_programs off only the decode-shaped steps that become graphs are recorded)
                wanted = rec.shape is not None and (self.config.use_programs or rec.wants_graph)
                ran = rec.replay(t_start, defer_update=forcing) if (wanted and rec.has_program) else None
                if ran is not None:      # the native engine ran the step (and, unless deferred, the update)
                    info.rows, info.seqs, ids = ran
                elif wanted:
                    layout, ids = rec.record(sampling)
                    info.rows, info.seqs = layout.rows, layout.seqs
                else:
                    with torch.cuda.stream(rec.stream):
                        ids = self._step_direct(info, sampling)
        if ids is not None:
            if forcing:
                ids = self._force(ids)
            self.core.update_sampled(ids, self.now())
        info.ms = (self.now() - t_start) * 1e3
        return info

    def _step_direct(self, info: StepInfo, sampling: int) -> np.ndarray:
        """The planned step through the model's parts, launch by launch; -> the sampled ids."""
        layout = self.core.build_batch_from_plan(self.runner.host_buffer())
        logits = self.runner.execute(layout)
        info.rows, info.seqs = layout.rows, layout.seqs
        if sampling:
            return self.sampler.sample_on_device(logits, self.runner.last_step.sampling_params())
        torch.cuda.current_stream().synchronize()
        return np.zeros(0, dtype=np.int32)

    def _force(self, ids: np.ndarray) -> np.ndarray:
        """Teacher forcing: the step's sampled ids are replaced by the tokens the request brought, and
        the logits they were sampled from are kept (src/main_correct.cpp:194-222 scores given tokens
        the same way, one whole sequence at a time)."""
        R = len(ids)
        if R == 0:
            return ids
        rows = self.runner.workspace.get("logits", (R, self.model.spec.vocab_size), torch.float32).cpu().numpy()
        out, k = ids.copy(), 0
        for p in self.core.plan():
            if not p.samples:
                continue
            given = self._forced.get(p.id)
            if given is not None:
                self._forced_logits[p.id][p.gen_index] = rows[k]
                out[k] = given[p.gen_index]
            k += 1
        return out

    def forced_logits(self, request_id: int) -> np.ndarray:
        """Of a request added with ``forced``: the logits each of its forced tokens was to be sampled
        from, [len(forced), vocab] (a row of NaN where none has been computed yet).  A finished
        request's logits are handed out once: the engine keeps nothing of it afterwards."""
        if request_id in self._forced:
            return self._forced_logits[request_id].copy()
        return self._forced_logits.pop(request_id)

    def run_until_idle(self, max_steps: int = 1 << 30) -> List[Finished]:
        done = []
        steps = 0
        while not self.idle() and steps < max_steps:
            self.step()
            done.extend(self.take_finished())
            steps += 1
        return done

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, temperature: float = 0.0,
                 seed: int = 0) -> List[List[int]]:
        """Runs the prompts together to completion; returns the generated ids per prompt (an empty
        list for a prompt that can never fit the pool)."""
        ids = [self.add_request(p, max_new_tokens, temperature, seed) for p in prompts]
        by_id = {f.id: f for f in self.run_until_idle()}
        return [by_id[i].generated if i in by_id else [] for i in ids]

    # ------------------------------------------------------------------------------ score
    def score(self, tokens: Sequence[int]) -> np.ndarray:
        """Teacher-forced logits [n, vocab] at every position of ``tokens``, through the real
        manager and pages (src/engine/engine.cpp:92-108)."""
        if self.core.prefix_caching:
            raise RuntimeError("score: disable prefix caching (every position is recomputed, which would rewrite shared pages)")
        sid = self._score_id
        self._score_id -= 1
        toks = [int(t) for t in tokens]
        self.core.seq_new(sid, toks)
        try:
            if not self.core.can_admit(sid):
                raise RuntimeError("score: the sequence does not fit in the KV pool")
            self.core.admit(sid)
            try:
                layout = self.core.build_batch([(sid, 0, len(toks), list(range(len(toks))))], self.runner.host_buffer())
                if self.recorded is None:
                    return self.runner.execute_to_host(layout)
                with torch.cuda.stream(self.recorded.stream):      # the stream every step of this engine runs on
                    return self.runner.execute_to_host(layout)
            finally:
                self.core.release(sid)
        finally:
            self.core.seq_delete(sid)

    # ------------------------------------------------------------------------------ info
    @property
    def num_blocks(self) -> int:
        return self.runner.num_blocks

    def bytes_per_block(self) -> int:
        return sum(s.bytes_per_block for s in self.runner.storages if hasattr(s, "bytes_per_block"))

    def cache_bytes(self) -> int:
        return sum(s.total_bytes for s in self.runner.storages)
