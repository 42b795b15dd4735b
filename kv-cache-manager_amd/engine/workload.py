"""Synthetic requests: Poisson arrivals, lognormal prompt and output lengths, an optional shared
prefix, optional lengths from a CSV.  Same knobs, clamping rules and defaults as the reference's
generator (src/sim/workload.h:14-27, src/sim/workload.cpp:64-125); the random streams are
NumPy's, so the individual draws differ from the reference's mt19937_64 ones.  Token ids are
uniform in [3, vocab) (ids 0..2 are avoided, workload.cpp:105); a shared prefix's tokens depend
on the prefix id only."""
import csv
import math
from dataclasses import dataclass
from typing import List

import numpy as np


@dataclass
class WorkloadConfig:
    num_requests: int = 1000
    arrival_rate: float = 0.0          # requests per second; <= 0: all arrive at t = 0
    prompt_mu: float = 5.0
    prompt_sigma: float = 1.0
    output_mu: float = 5.3
    output_sigma: float = 0.9
    min_prompt: int = 4
    max_prompt: int = 1024
    min_output: int = 4
    max_output: int = 1024
    max_seq_len: int = 2048
    shared_frac: float = 0.0
    shared_len: int = 0
    num_shared_prefixes: int = 1
    lengths_csv: str = ""
    vocab: int = 32000
    seed: int = 1

    @classmethod
    def from_args(cls, a) -> "WorkloadConfig":
        c = cls()
        c.num_requests = a.i32("requests", c.num_requests)
        c.arrival_rate = a.f64("rate", c.arrival_rate)
        c.prompt_mu, c.prompt_sigma = a.f64("prompt-mu", c.prompt_mu), a.f64("prompt-sigma", c.prompt_sigma)
        c.output_mu, c.output_sigma = a.f64("output-mu", c.output_mu), a.f64("output-sigma", c.output_sigma)
        c.min_prompt, c.max_prompt = a.i32("min-prompt", c.min_prompt), a.i32("max-prompt", c.max_prompt)
        c.min_output, c.max_output = a.i32("min-output", c.min_output), a.i32("max-output", c.max_output)
        c.max_seq_len = a.i32("max-seq-len", c.max_seq_len)
        c.shared_frac, c.shared_len = a.f64("shared-frac", c.shared_frac), a.i32("shared-len", c.shared_len)
        c.num_shared_prefixes = a.i32("num-prefixes", c.num_shared_prefixes)
        c.lengths_csv = a.str("lengths-csv", c.lengths_csv)
        c.seed = a.i64("seed", c.seed)
        if a.has("prompt-len"):                      # fixed lengths override the distributions
            n = a.i32("prompt-len", 0)
            c.prompt_sigma, c.prompt_mu, c.min_prompt, c.max_prompt = 0.0, math.log(max(n, 1)), n, n
        if a.has("output-len"):
            n = a.i32("output-len", 0)
            c.output_sigma, c.output_mu, c.min_output, c.max_output = 0.0, math.log(max(n, 1)), n, n
        return c

    def describe(self) -> str:
        return (f"requests={self.num_requests} rate={self.arrival_rate:g} prompt~LN({self.prompt_mu:g},{self.prompt_sigma:g}) "
                f"output~LN({self.output_mu:g},{self.output_sigma:g}) shared_frac={self.shared_frac:g} "
                f"shared_len={self.shared_len} max_seq_len={self.max_seq_len} seed={self.seed}")


@dataclass
class Request:
    id: int
    arrival: float
    prompt_len: int      # including the shared prefix
    output_len: int
    prefix_id: int       # -1: no shared prefix


def _load_lengths(path):
    rows = []
    with open(path) as f:
        for rec in csv.reader(f):
            try:
                p, o = int(rec[0]), int(rec[1])
            except (ValueError, IndexError):
                continue
            if p > 0 and o > 0:
                rows.append((p, o))
    if not rows:
        raise ValueError(f"no rows in lengths csv: {path}")
    return rows


def generate_workload(c: WorkloadConfig) -> List[Request]:
    rng = np.random.default_rng(c.seed)
    table = _load_lengths(c.lengths_csv) if c.lengths_csv else None
    out, t, next_prefix = [], 0.0, 0
    for i in range(c.num_requests):
        if c.arrival_rate > 0:
            t += rng.exponential(1.0 / c.arrival_rate)
        if table:
            p, o = table[int(rng.integers(0, len(table)))]
        else:
            p = int(round(rng.lognormal(c.prompt_mu, max(c.prompt_sigma, 1e-9))))
            o = int(round(rng.lognormal(c.output_mu, max(c.output_sigma, 1e-9))))
        p = min(max(p, c.min_prompt), c.max_prompt)
        o = min(max(o, c.min_output), c.max_output)
        prefix = -1
        if c.shared_len > 0 and rng.random() < c.shared_frac:
            prefix = next_prefix % max(1, c.num_shared_prefixes)
            next_prefix += 1
            p += c.shared_len
        p = min(p, c.max_seq_len - 1)
        o = max(1, min(o, c.max_seq_len - p))
        out.append(Request(i, t, p, o, prefix))
    return out


def make_prompt_tokens(r: Request, c: WorkloadConfig) -> List[int]:
    toks: List[int] = []
    if r.prefix_id >= 0:
        prng = np.random.default_rng([c.seed, 0xABCDEF, r.prefix_id])
        toks = prng.integers(3, c.vocab, size=min(c.shared_len, r.prompt_len)).tolist()
    rng = np.random.default_rng([c.seed, 0x1234567, r.id])
    toks += rng.integers(3, c.vocab, size=r.prompt_len - len(toks)).tolist()
    return toks
