"""The command-line tools as a user runs them, on tiny models: they finish, print what they
promise and return the exit codes the reference's tools use (src/main_bench.cpp,
src/main_correct.cpp, src/main_kernel_bench.cpp)."""
import csv
import os
import subprocess
import sys

import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(tool, *args, timeout=110):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", tool), *args], capture_output=True, text=True,
                          timeout=timeout)


def test_kvkernel_writes_one_row_per_variant(tmp_path):
    out = str(tmp_path / "k.csv")
    p = _run("kvkernel", "--ctx", "100,300", "--batch", "2", "--block-size", "16", "--iters", "3", "--out", out)
    assert p.returncode == 0, p.stderr
    rows = list(csv.DictReader(open(out)))
    assert len(rows) == 12 and {r["variant"] for r in rows} == {"paged-v1", "contiguous-v1", "paged-v2", "contiguous-v2",
                                                                 "paged-fused", "contiguous-fused"}
    for r in rows:
        assert float(r["us"]) > 0 and float(r["gbps"]) > 0 and int(r["regs"]) > 0 and int(r["wgs_per_cu"]) >= 1
    assert "unsupported" not in p.stdout
    # a shape the partitioned kernel does not take is reported, not silently replaced
    p = _run("kvkernel", "--ctx", "64", "--batch", "1", "--heads", "12", "--kv-heads", "1", "--iters", "1")
    assert p.returncode == 0 and p.stdout.count("unsupported") == 4


def test_kvbench_runs_a_small_workload(tmp_path):
    summary = str(tmp_path / "s.csv")
    p = _run("kvbench", "--random-weights", "--sizes", "tiny-a", "--dtype", "bf16", "--requests", "6", "--prompt-len", "9",
             "--output-len", "5", "--max-seq-len", "64", "--num-blocks", "32", "--warmup", "1", "--summary", summary)
    assert p.returncode == 0, p.stderr + p.stdout
    rows = list(csv.DictReader(open(summary)))
    assert len(rows) == 1


def test_kvcorrect_passes_on_a_tiny_model(tmp_path):
    d = str(tmp_path / "m")
    H.make_model_dir(d, H.CONFIGS["A"], H.WEIGHT_SEED["A"], torch.bfloat16)
    p = _run("kvcorrect", "--model", d, "--dtype", "bf16", "--max-seq-len", "128", "--num-blocks", "64", "--steps", "8")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "ALL CHECKS PASSED" in p.stdout
    # the yardstick of that kind of run, kept in the reference's container, serves a later run as --refs
    refs = str(tmp_path / "refs.bin")
    p = _run("kvcorrect", "--model", d, "--dtype", "bf16", "--max-seq-len", "128", "--num-blocks", "64", "--steps", "8",
             "--write-refs", refs)
    assert p.returncode == 0 and os.path.getsize(refs) > 16, p.stdout + p.stderr
    p = _run("kvcorrect", "--model", d, "--dtype", "bf16", "--max-seq-len", "128", "--num-blocks", "64", "--refs", refs)
    assert p.returncode == 0 and "8 reference prompts, 8 steps" in p.stdout, p.stdout + p.stderr
