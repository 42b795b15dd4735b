"""Serving metrics: time to first token, end-to-end latency, time per output token, throughput;
the same quantities, percentile rule and CSV columns as the reference
(src/engine/metrics.h:12-34, src/engine/metrics.cpp:11-96)."""
import math
import os
from dataclasses import dataclass, field, fields
from typing import List


def percentile(values, p: float) -> float:
    """Linear interpolation between order statistics (src/engine/metrics.cpp:11-17)."""
    if not values:
        return 0.0
    v = sorted(values)
    idx = p * (len(v) - 1)
    lo, hi = int(math.floor(idx)), int(math.ceil(idx))
    return v[lo] + (v[hi] - v[lo]) * (idx - lo)


@dataclass
class BenchSummary:
    policy: str = ""
    block_size: int = 0
    num_blocks: int = 0
    pool_gb: float = 0.0
    rate: float = 0.0
    shared_frac: float = 0.0
    requests: int = 0
    completed: int = 0
    rejected: int = 0
    wall_s: float = 0.0
    output_tokens: int = 0
    prompt_tokens: int = 0
    out_tok_s: float = 0.0
    total_tok_s: float = 0.0
    req_s: float = 0.0
    ttft_mean: float = 0.0
    ttft_p50: float = 0.0
    ttft_p95: float = 0.0
    ttft_p99: float = 0.0
    e2e_p50: float = 0.0
    e2e_p95: float = 0.0
    e2e_p99: float = 0.0
    tpot_mean_ms: float = 0.0
    mean_batch: float = 0.0
    max_batch: int = 0
    preemptions: int = 0
    steps: int = 0
    mean_step_ms: float = 0.0
    prefill_tokens: int = 0
    prefill_saved: int = 0
    prefix_hit_rate: float = 0.0
    evictions: int = 0
    peak_blocks: int = 0
    peak_kv_gb: float = 0.0
    gpu_used_gb: float = 0.0


class MetricsCollector:
    def __init__(self):
        self.ttft: List[float] = []
        self.e2e: List[float] = []
        self.tpot: List[float] = []
        self.out_tokens = 0
        self.prompt_tokens = 0
        self.rejected = 0

    def add_finished(self, f):
        """f: cache.manager.Finished."""
        if f.first_token < 0:
            self.rejected += 1
            return
        self.ttft.append(f.first_token - f.arrival)
        self.e2e.append(f.finished - f.arrival)
        out = len(f.tokens) - f.prompt_len
        if out > 1:
            self.tpot.append((f.finished - f.first_token) / (out - 1))
        self.out_tokens += out
        self.prompt_tokens += f.prompt_len

    def count(self) -> int:
        return len(self.ttft)

    def finalize(self, s: BenchSummary, wall_s: float):
        mean = lambda v: sum(v) / len(v) if v else 0.0
        s.completed, s.rejected, s.wall_s = len(self.ttft), self.rejected, wall_s
        s.output_tokens, s.prompt_tokens = self.out_tokens, self.prompt_tokens
        s.out_tok_s = self.out_tokens / wall_s if wall_s > 0 else 0.0
        s.total_tok_s = (self.out_tokens + self.prompt_tokens) / wall_s if wall_s > 0 else 0.0
        s.req_s = s.completed / wall_s if wall_s > 0 else 0.0
        s.ttft_mean = mean(self.ttft)
        s.ttft_p50, s.ttft_p95, s.ttft_p99 = (percentile(self.ttft, p) for p in (0.5, 0.95, 0.99))
        s.e2e_p50, s.e2e_p95, s.e2e_p99 = (percentile(self.e2e, p) for p in (0.5, 0.95, 0.99))
        s.tpot_mean_ms = 1e3 * mean(self.tpot)


def print_summary(s: BenchSummary):
    print(f"[{s.policy}] B={s.block_size} blocks={s.num_blocks} ({s.pool_gb:.2f} GB) rate={s.rate:g} shared={s.shared_frac:g}")
    print(f"  completed {s.completed}/{s.requests} (rejected {s.rejected}) in {s.wall_s:.2f}s, {s.steps} steps ({s.mean_step_ms:.2f} ms/step)")
    print(f"  throughput: {s.out_tok_s:.1f} out tok/s, {s.total_tok_s:.1f} total tok/s, {s.req_s:.2f} req/s")
    print(f"  TTFT p50/p95/p99 = {s.ttft_p50:.3f} / {s.ttft_p95:.3f} / {s.ttft_p99:.3f} s   "
          f"E2E p50/p95/p99 = {s.e2e_p50:.3f} / {s.e2e_p95:.3f} / {s.e2e_p99:.3f} s")
    print(f"  TPOT mean {s.tpot_mean_ms:.2f} ms   batch mean {s.mean_batch:.1f} max {s.max_batch}   preemptions {s.preemptions}")
    print(f"  prefill tokens {s.prefill_tokens} (saved {s.prefill_saved}, block hit rate {100 * s.prefix_hit_rate:.1f}%, "
          f"evictions {s.evictions})")
    print(f"  peak KV blocks {s.peak_blocks} ({s.peak_kv_gb:.3f} GB), GPU memory used {s.gpu_used_gb:.2f} GB")


def append_bench_csv(path: str, s: BenchSummary):
    names = [f.name for f in fields(BenchSummary)]
    fresh = not os.path.exists(path) or os.path.getsize(path) == 0
    with open(path, "a") as f:
        if fresh:
            f.write(",".join(names) + "\n")
        f.write(",".join(f"{getattr(s, n):.4f}" if isinstance(getattr(s, n), float) else str(getattr(s, n)) for n in names) + "\n")
