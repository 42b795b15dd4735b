"""bench.py's contract with whoever runs it: one GPU only, one JSON line, a flat configuration."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _run(*args, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True, env=e, timeout=600)


def test_more_than_one_gpu_is_refused_with_one_line_and_exit_code_2():
    r = _run("--gpus", "2")
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout
    r = _run(env={"WORLD_SIZE": "4"})
    assert r.returncode == 2 and len(r.stdout.strip().splitlines()) == 1


def test_unknown_sizes_and_a_context_limit_that_cannot_hold_the_run_are_refused():
    r = _run("--sizes", "no-such-model")
    assert r.returncode == 2 and "unknown --sizes" in r.stdout
    r = _run("--prompt-len", "2040", "--context-limit", "2048")
    assert r.returncode == 2 and "does not fit" in r.stdout


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_fields():
    r = _run("--layers", "2", "--steps", "6", "--warmup", "2", "--batch", "2", "--prompt-len", "64")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "points", "prefill"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 6 and d["warmup"] == 2 and d["higher_is_better"] is True
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_full"] == 22 and cfg["global_batch"] == 2
    assert abs(d["value"] - 2 * 1e3 / d["ms_per_step"]) < 0.01 * d["value"]
    assert d["prefill"]["tokens"] == 2048 and 0 < d["prefill"]["frac"] < 1
    assert d["roofline"]["bound"] == "hbm" and d["roofline"]["peak"] == 8000.0
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / d["roofline"]["peak"]) < 1e-3
    assert {"decode_b1", "decode_b64"} <= set(d["points"])


def test_trace_run_scheduled_refuses_bad_requests_before_it_loads_a_model(tmp_path):
    """The second mode of bin/trace_run reads every request first: what a line gets wrong ends the program with
    one line on stderr and exit code 1, with no model loaded (so this runs without a GPU)."""
    tool = os.path.join(ROOT, "bin", "trace_run")
    good = '{"id": "a", "prompt": [1, 2], "forced": [3]}'
    for lines, what in (([good, '{"id": "a", "prompt": [4], "forced": [5]}'], "appears twice"),
                        (['{"id": "x/y", "prompt": [1], "forced": [2]}'], "name a file"),
                        (['{"id": "b", "prompt": [], "forced": [2]}'], "at least one token"),
                        (['{"id": "b", "prompt": [1]}'], "missing key"),
                        (["not json"], "line 1")):
        r = subprocess.run([sys.executable, tool, "--scheduled", "--model", str(tmp_path / "none"), "--out", str(tmp_path / "o")],
                           input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=120)
        assert r.returncode == 1 and "trace_run: input line" in r.stderr and what in r.stderr, (lines, r.returncode, r.stderr[-300:])
        assert len([l for l in r.stderr.splitlines() if l.startswith("trace_run:")]) == 1
    r = subprocess.run([sys.executable, tool, "--scheduled", "--out", str(tmp_path / "o")], input="", capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "give --model DIR and --out DIR" in r.stderr
