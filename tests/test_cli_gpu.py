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


def test_kvgen_prints_the_generated_ids_of_given_prompts(tmp_path):
    """A model folder and prompts as token ids in, one line of generated ids per prompt out: the same ids
    the plain implementation generates (up to near ties of its two best scores)."""
    import plain_llama as plain
    d = str(tmp_path / "m")
    H.make_model_dir(d, H.CONFIGS["A"], H.WEIGHT_SEED["A"], torch.float32)
    prompts = [[5, 17, 3, 200, 41], [9, 9, 1], [100]]
    (tmp_path / "more.txt").write_text("7 8 9 10\n")
    p = _run("kvgen", "--model", d, "--dtype", "fp32", "--prompt-ids", "5,17,3,200,41", "--prompt-ids=9,9,1", "--prompt-ids", "100",
             "--prompts-file", str(tmp_path / "more.txt"), "--max-new-tokens", "6", "--max-seq-len", "64", "--num-blocks", "16",
             "--dump-tables")
    assert p.returncode == 0, p.stderr
    lines = p.stdout.strip("\n").split("\n")
    assert len(lines) == 4
    pm = plain.load_model_dir(d, None)
    for prompt, line in zip(prompts + [[7, 8, 9, 10]], lines):
        got = [int(t) for t in line.split()]
        want, margins = pm.generate(prompt, 6)
        first = next((k for k in range(6) if got[k] != want[k]), None)
        assert len(got) == 6 and (first is None or margins[first] < 1e-4), (prompt, got, want)
    import json
    dumps = [json.loads(l) for l in p.stderr.split("\n") if l.startswith("{")]
    assert dumps and dumps[0]["step"] == 0 and set(dumps[0]["tables"]) == {"0", "1", "2", "3"}
    assert all(len(g) == 1 and len(g[0]) == 1 for g in dumps[0]["tables"].values())       # one group, one page each
    # temperature sampling with a seed is reproducible, and differs from greedy somewhere
    a = _run("kvgen", "--model", d, "--dtype", "fp32", "--prompt-ids", "5,17,3", "--max-new-tokens", "12", "--temperature", "1.5",
             "--sampler-seed", "7", "--max-seq-len", "64", "--num-blocks", "16")
    b = _run("kvgen", "--model", d, "--dtype", "fp32", "--prompt-ids", "5,17,3", "--max-new-tokens", "12", "--temperature", "1.5",
             "--sampler-seed", "7", "--max-seq-len", "64", "--num-blocks", "16")
    g = _run("kvgen", "--model", d, "--dtype", "fp32", "--prompt-ids", "5,17,3", "--max-new-tokens", "12", "--max-seq-len", "64",
             "--num-blocks", "16")
    assert a.returncode == b.returncode == g.returncode == 0 and a.stdout == b.stdout != g.stdout
    # what it cannot run: one line, exit code 1
    bad = _run("kvgen", "--model", d, "--prompt-ids", "5,99999")
    assert bad.returncode == 1 and "outside the vocabulary" in bad.stderr
    assert _run("kvgen", "--model", d).returncode == 1
