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
        self._t0 = time.perf_counter()
        self.config = self.runner.engine_config      # as built (max_seq_len within the model's range)
        # Recorded steps (graphs) replay a fixed launch sequence: only for models whose parts all
        # declare that their launches depend on the step's shape alone (Part.capturable).
        self.decode_graphs = None
        self.programs = None
        if self.config.use_graphs and self.model.capturable:
            from .graphs import DecodeGraphs
            self.decode_graphs = DecodeGraphs(self)

    # ------------------------------------------------------------------------------ clock
    def now(self) -> float:
        return time.perf_counter() - self._t0

    def reset_clock(self):
        self._t0 = time.perf_counter()

    # --------------------------------------------------------------------------- requests
    def add_request(self, tokens: Sequence[int], max_new_tokens: int, temperature: float = 0.0, seed: int = 0,
                    request_id: Optional[int] = None, arrival: Optional[float] = None) -> int:
        if request_id is None:
            request_id = self._next_id
        self._next_id = max(self._next_id, request_id + 1)
        toks = [int(t) for t in tokens]
        V = self.model.spec.vocab_size
        if not toks:
            raise ValueError("a request needs at least one token")
        if min(toks) < 0 or max(toks) >= V:
            raise ValueError(f"token id outside the vocabulary of {V}")
        self.core.sched_add(request_id, toks, int(max_new_tokens), float(temperature), int(seed),
                            self.now() if arrival is None else arrival)
        return request_id

    add = add_request

    def idle(self) -> bool:
        return self.core.idle()

    def take_finished(self) -> List[Finished]:
        return self.core.take_finished()

    # ------------------------------------------------------------------------------- step
    def step(self) -> StepInfo:
        info = StepInfo()
        t_start = self.now()
        n, info.prefill_tokens, info.decode_seqs, sampling, decode_shaped = self.core.schedule_summary(t_start)
        if n == 0:
            return info
        if self.decode_graphs is not None and decode_shaped and self.decode_graphs.fits(n):
            ids = self.decode_graphs.run(n)
            info.rows = info.seqs = n
        else:
            layout = self.core.build_batch_from_plan(self.runner.host_buffer())
            logits = self.runner.execute(layout)
            info.rows, info.seqs = layout.rows, layout.seqs
            ids = np.zeros(0, dtype=np.int32)
            if sampling:
                ids = self.sampler.sample_on_device(logits, self.runner.last_step.sampling_params())
            else:
                torch.cuda.current_stream().synchronize()
        t_end = self.now()
        self.core.update_sampled(ids, t_end)
        info.ms = (t_end - t_start) * 1e3
        return info

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
