"""The serving tools' workload generator and metrics (no GPU): the reference's knobs, clamping
rules and CSV columns (src/sim/workload.cpp:64-125, src/engine/metrics.cpp:11-96,
results/bench_capacity.csv for the column names)."""
import math
from types import SimpleNamespace

import numpy as np
import pytest

from kvcm_amd.cli.args import Args
from kvcm_amd.engine.metrics import BenchSummary, MetricsCollector, append_bench_csv, percentile
from kvcm_amd.engine.workload import WorkloadConfig, generate_workload, make_prompt_tokens


def test_workload_clamps_lengths_as_the_reference_does():
    c = WorkloadConfig(num_requests=500, max_seq_len=300, max_prompt=1024, max_output=1024, seed=5)
    reqs = generate_workload(c)
    assert len(reqs) == 500 and all(r.arrival == 0.0 for r in reqs)                 # rate 0: a burst
    assert all(c.min_prompt <= r.prompt_len <= c.max_seq_len - 1 for r in reqs)     # prompt <= max_seq_len - 1
    assert all(1 <= r.output_len and r.prompt_len + r.output_len <= c.max_seq_len for r in reqs)
    assert generate_workload(c) == reqs                                             # the seed fixes everything
    assert generate_workload(WorkloadConfig(num_requests=500, max_seq_len=300, seed=6)) != reqs
    med = np.median([r.prompt_len for r in generate_workload(WorkloadConfig(num_requests=4000, seed=1))])
    assert abs(med - math.exp(5.0)) < 15                                            # lognormal(5, 1): median e^5 = 148


def test_workload_arrivals_prefixes_and_fixed_lengths():
    c = WorkloadConfig(num_requests=2000, arrival_rate=50.0, shared_frac=0.5, shared_len=64, num_shared_prefixes=3, seed=2)
    reqs = generate_workload(c)
    gaps = np.diff([0.0] + [r.arrival for r in reqs])
    assert (gaps >= 0).all() and abs(gaps.mean() - 1 / 50.0) < 0.003                 # Poisson arrivals at 50 / s
    with_prefix = [r for r in reqs if r.prefix_id >= 0]
    assert 0.4 < len(with_prefix) / len(reqs) < 0.6 and {r.prefix_id for r in with_prefix} == {0, 1, 2}
    a, b = [r for r in with_prefix if r.prefix_id == 1][:2]
    ta, tb = make_prompt_tokens(a, c), make_prompt_tokens(b, c)
    assert len(ta) == a.prompt_len and ta[:64] == tb[:64] and ta[64:70] != tb[64:70]  # the prefix depends on its id only
    assert min(ta) >= 3 and max(ta) < c.vocab                                       # ids 0..2 are avoided
    other = make_prompt_tokens([r for r in with_prefix if r.prefix_id == 2][0], c)
    assert other[:64] != ta[:64]
    fixed = WorkloadConfig.from_args(Args(["--requests", "7", "--prompt-len", "33", "--output-len", "5", "--seed", "9"]))
    assert [(r.prompt_len, r.output_len) for r in generate_workload(fixed)] == [(33, 5)] * 7


def test_workload_lengths_from_a_csv(tmp_path):
    path = tmp_path / "lengths.csv"
    path.write_text("prompt,output\n10,3\n200,40\nbad,row\n0,5\n")
    reqs = generate_workload(WorkloadConfig(num_requests=50, lengths_csv=str(path), seed=3))
    assert {(r.prompt_len, r.output_len) for r in reqs} == {(10, 4), (200, 40)}       # min_output 4 still clamps
    empty = tmp_path / "none.csv"
    empty.write_text("prompt,output\n")
    with pytest.raises(ValueError, match="no rows"):
        generate_workload(WorkloadConfig(num_requests=1, lengths_csv=str(empty)))


def test_percentile_interpolates_between_order_statistics():
    assert percentile([], 0.5) == 0.0
    assert percentile([4.0], 0.99) == 4.0
    assert percentile([1.0, 2.0, 3.0, 4.0], 0.5) == 2.5
    assert percentile([3.0, 1.0, 2.0], 0.95) == pytest.approx(2.9)


def test_metrics_of_finished_requests_and_the_csv_columns(tmp_path):
    mc = MetricsCollector()
    done = [SimpleNamespace(arrival=0.0, first_token=0.5, finished=2.5, tokens=list(range(15)), prompt_len=10),   # 5 out
            SimpleNamespace(arrival=1.0, first_token=1.25, finished=1.25, tokens=list(range(4)), prompt_len=3),   # 1 out: no TPOT
            SimpleNamespace(arrival=2.0, first_token=-1.0, finished=2.0, tokens=[1, 2], prompt_len=2)]            # rejected
    for f in done:
        mc.add_finished(f)
    s = BenchSummary(policy="paged", requests=3)
    mc.finalize(s, wall_s=4.0)
    assert (s.completed, s.rejected, s.output_tokens, s.prompt_tokens) == (2, 1, 6, 13)
    assert s.out_tok_s == 1.5 and s.total_tok_s == 19 / 4 and s.req_s == 0.5
    assert s.ttft_mean == pytest.approx(0.375) and s.ttft_p50 == pytest.approx(0.375)
    assert s.e2e_p99 == pytest.approx(0.25 + 0.99 * 2.25)
    assert s.tpot_mean_ms == pytest.approx(1e3 * 2.0 / 4)                            # (finished - first) / (out - 1)
    path = str(tmp_path / "summary.csv")
    append_bench_csv(path, s)
    append_bench_csv(path, s)
    lines = open(path).read().splitlines()
    assert len(lines) == 3 and lines[1] == lines[2]
    assert lines[0].split(",")[:13] == ["policy", "block_size", "num_blocks", "pool_gb", "rate", "shared_frac", "requests",
                                        "completed", "rejected", "wall_s", "output_tokens", "prompt_tokens", "out_tok_s"]
    assert lines[0].split(",")[-3:] == ["peak_blocks", "peak_kv_gb", "gpu_used_gb"] and len(lines[0].split(",")) == 35


def test_command_line_parsing_follows_the_reference(capsys):
    """--key=value, --key value and bare --flag, typed getters with defaults, and a warning for a flag
    that nobody read (src/common/args.h:12-58)."""
    a = Args(["--requests=12", "--rate", "2.5", "--prefix", "--policy", "paged", "--typo", "1"])
    assert a.i32("requests", 0) == 12 and a.f64("rate", 0.0) == 2.5 and a.flag("prefix") and a.str("policy", "x") == "paged"
    assert a.i32("block-size", 16) == 16 and not a.flag("no-graphs") and a.has("rate") and not a.has("seed")
    a.warn_unused()
    assert "unused flag --typo" in capsys.readouterr().err
    with pytest.raises(ValueError, match="bad argument"):
        Args(["requests", "3"])
