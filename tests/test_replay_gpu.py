"""The engine against the plain implementation, in 32-bit and in bfloat16, for every way of
cutting and batching the same requests: whole; most in one step and the last 32 tokens one by
one; portions of changing size down to two tokens; up to four live requests mixed, with so few
pages that they are used again.  A difference that shows in one schedule only is a fault of the
cache or the batch: the assertion names the first wrong (request, position)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"A": [7, 70, 13, 45, 5, 100, 33, 64], "B": [1, 9, 17, 33, 40, 130, 2, 65], "C": [50, 3, 97, 16, 31],
           "D": [300, 20, 1100, 65, 257], "E": [40, 3, 300, 17, 129]}


def tolerance(dtype, ref):
    scale = max(1.0, max(float(np.abs(r).max()) for r in ref.values()))
    # 32-bit: rounding of sums only.  bfloat16 against the plain implementation that rounds at the
    # same places: what is left is a rounding that falls the other way now and then.
    return (1e-5 if dtype == "float32" else 1e-2) * scale


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    """model folder, requests, plain logits and one replayer per (config, dtype)."""
    from kvcm_amd.engine.replay import TraceReplayer
    out = {}
    for name, raw in H.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            d = str(tmp_path_factory.mktemp(f"model_{name}_{dtype}"))
            H.make_model_dir(d, raw, H.WEIGHT_SEED[name], torch.float32 if dtype == "float32" else torch.bfloat16,
                             sharpen=H.SHARPEN[name])
            reqs = H.requests_for(raw, LENGTHS[name], seed=1 + H.WEIGHT_SEED[name])
            ref, _ = H.plain_logits(d, reqs, bf16=dtype == "bfloat16")
            rp = TraceReplayer(d, dtype, max_tokens=H.tokens_needed(reqs), block_size=H.BLOCK_SIZE[name])
            out[(name, dtype)] = (d, reqs, ref, rp)
    return out


CASES = [(n, d) for n in ("A", "B", "C", "D", "E") for d in ("float32", "bfloat16")]


def check(setups, case, steps):
    d, reqs, ref, rp = setups[case]
    got = H.replay(rp, steps, reqs)
    assert all(not np.isnan(g).any() for g in got.values()), "a wanted position got no logits"
    bad = H.first_difference(got, ref, tolerance(case[1], ref))
    assert bad is None, f"first wrong logits at request {bad[0]} position {bad[1]}: error {bad[2]:.3g}"
    assert rp.core.blocks_in_use() == 0, "pages were not given back"
    return got


@pytest.mark.parametrize("case", CASES)
def test_each_request_alone_and_whole(setups, case):
    check(setups, case, H.schedule_whole(setups[case][1]))


@pytest.mark.parametrize("case", CASES)
def test_last_32_tokens_one_by_one(setups, case):
    check(setups, case, H.schedule_tail_singly(setups[case][1], 32))


@pytest.mark.parametrize("case", CASES)
def test_portions_of_changing_size(setups, case):
    check(setups, case, H.schedule_portions(setups[case][1]))


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("seed", [0, 1])
def test_mixed_batches_with_reused_pages(setups, case, seed):
    d, reqs, ref, rp = setups[case]
    steps = H.schedule_mixed(reqs, seed=seed)
    assert max(len(s["entries"]) for s in steps) > 1
    assert any(len(e["tokens"]) > 1 for s in steps if len(s["entries"]) > 1 for e in s["entries"])
    check(setups, case, steps)


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_32bit_logits_do_not_depend_on_the_cutting(setups, name):
    """In 32-bit every kernel computes a row by a fixed sequence of operations, so the cuttings
    agree to the last bit, not just within rounding."""
    case = (name, "float32")
    whole = check(setups, case, H.schedule_whole(setups[case][1]))
    for steps in (H.schedule_tail_singly(setups[case][1]), H.schedule_portions(setups[case][1]),
                  H.schedule_mixed(setups[case][1], seed=3)):
        got = H.replay(setups[case][3], steps, setups[case][1])
        for rid in whole:
            diff = np.nonzero((got[rid] != whole[rid]).any(axis=1))[0]
            assert len(diff) == 0, f"request {rid}: position {diff[0]} differs between cuttings"


@pytest.mark.parametrize("case", CASES)
def test_first_tokens_of_a_sequence(setups, case):
    d, reqs, ref, rp = setups[case]
    first = {rid: t[:3] for rid, t in reqs.items()}
    steps = [{"step": k, "entries": [{"id": rid, "tokens": [t[0]], "want": [0]}], "end": []}
             for k, (rid, t) in enumerate(list(first.items())[:4])]
    steps += [{"step": 10 + k, "entries": [{"id": rid, "tokens": t[1:], "want": list(range(len(t) - 1))}], "end": [rid]}
              for k, (rid, t) in enumerate(list(first.items())[:4]) if len(t) > 1]
    for k, (rid, t) in enumerate(list(first.items())[:4]):
        if len(t) == 1:
            steps.append({"step": 20 + k, "entries": [], "end": [rid]})
    sub = {rid: first[rid] for rid in list(first)[:4]}
    got = H.replay(rp, steps, sub)
    tol = tolerance(case[1], ref)
    for rid, t in sub.items():
        assert np.abs(got[rid] - ref[rid][:len(t)]).max() <= tol
    assert rp.core.blocks_in_use() == 0


def _config(V, H_, I, L, nh, nkv, hd, theta=10000.0, eps=1e-5, tied=False):
    return dict(architectures=["LlamaForCausalLM"], vocab_size=V, hidden_size=H_, intermediate_size=I, num_hidden_layers=L,
                num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, max_position_embeddings=1024, rope_theta=theta,
                rms_norm_eps=eps, tie_word_embeddings=tied)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("raw", [_config(301, 72, 104, 2, 6, 2, 24, theta=5e5, eps=1e-6), _config(500, 80, 112, 1, 5, 1, 40, tied=True),
                                 _config(259, 128, 192, 1, 4, 2, 120), _config(263, 96, 136, 1, 2, 2, 248),
                                 _config(101, 99, 77, 2, 3, 1, 32, theta=5e5, eps=1e-6)],
                         ids=["hd24", "hd40", "hd120", "hd248", "odd_widths"])
def test_head_sizes_in_steps_of_8_and_odd_widths(raw, dtype, tmp_path):
    """The configuration takes head sizes in steps of 8 up to 256; those that are no multiple of 16 run through
    the general kernels, whole and mixed with reused pages like every other size.  So does a model whose width,
    feed-forward width and vocabulary are odd numbers (no vector load fits a row)."""
    from kvcm_amd.engine.replay import TraceReplayer
    d = str(tmp_path)
    H.make_model_dir(d, raw, 3, torch.float32 if dtype == "float32" else torch.bfloat16, sharpen=6.0)
    reqs = H.requests_for(raw, [40, 3, 300, 17], seed=4)
    ref, _ = H.plain_logits(d, reqs, bf16=dtype == "bfloat16")
    rp = TraceReplayer(d, dtype, max_tokens=H.tokens_needed(reqs), block_size=16)
    for steps in (H.schedule_whole(reqs), H.schedule_tail_singly(reqs, 32), H.schedule_mixed(reqs, seed=1)):
        got = H.replay(rp, steps, reqs)
        bad = H.first_difference(got, ref, tolerance(dtype, ref))
        assert bad is None, f"first wrong logits at request {bad[0]} position {bad[1]}: error {bad[2]:.3g}"
    assert rp.core.blocks_in_use() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(setups, dtype):
    """One token at a time from the very first, across many page edges."""
    d, reqs, ref, rp = setups[("A", dtype)]
    rid = "r5"
    toks = reqs[rid]
    steps = [{"step": i, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
              "end": [rid] if i == len(toks) - 1 else []} for i in range(len(toks))]
    got = H.replay(rp, steps, {rid: toks})
    bad = H.first_difference(got, {rid: ref[rid]}, tolerance(dtype, ref))
    assert bad is None, f"first wrong logits at position {bad[1]}: error {bad[2]:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_beyond_2048_tokens_of_context(setups, dtype):
    """A few rows with a long context: in bfloat16 the decode kernel cuts such contexts into parts
    (nine chunks here) that a second launch merges."""
    from kvcm_amd.engine.replay import TraceReplayer
    d, _, ref_all, _ = setups[("D", dtype)]
    raw = H.TINY_D
    toks = np.random.default_rng(77).integers(0, raw["vocab_size"], size=2150).tolist()
    ref, _ = H.plain_logits(d, {"long": toks}, bf16=dtype == "bfloat16")
    rp = TraceReplayer(d, dtype, max_tokens=2176, block_size=H.BLOCK_SIZE["D"])
    ops, bounds = rp.runner.ops, []
    inner = ops.attention_decode_fused
    if dtype == "bfloat16":
        ops.attention_decode_fused = lambda *a, **k: (bounds.append(k.get("max_context", 0)), inner(*a, **k))[1]
    try:
        steps = [{"step": 0, "entries": [{"id": "long", "tokens": toks[:2100], "want": [2099]}], "end": []}]
        steps += [{"step": i - 2099, "entries": [{"id": "long", "tokens": [toks[i]], "want": [0]}],
                   "end": ["long"] if i == 2149 else []} for i in range(2100, 2150)]
        got = H.replay(rp, steps, {"long": toks})
    finally:
        ops.attention_decode_fused = inner
    tol = tolerance(dtype, ref)
    err = np.abs(got["long"][2099:] - ref["long"][2099:]).max(axis=1)
    assert (err <= tol).all(), f"first wrong logits at position {2099 + int(np.nonzero(err > tol)[0][0])}: {err.max():.3g}"
    if dtype == "bfloat16":
        assert len(bounds) == 50 * raw["num_hidden_layers"] and min(bounds) > 2048
        nh, nkv, hd = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
        assert ops.attention_decode_fused_scratch(1, nh, nkv, hd, min(bounds)) > 0       # in parts


def test_stale_pages_do_not_leak_into_a_new_request(setups):
    """A request that inherits pages full of another request's keys must not see them."""
    d, reqs, ref, rp = setups[("B", "float32")]
    long_id, short_id = "r5", "r2"           # 130 tokens, then 17 tokens on the same pages
    steps = [{"step": 0, "entries": [{"id": long_id, "tokens": reqs[long_id], "want": []}], "end": [long_id]},
             {"step": 1, "entries": [{"id": short_id, "tokens": reqs[short_id][:9], "want": list(range(9))}], "end": []},
             {"step": 2, "entries": [{"id": short_id, "tokens": reqs[short_id][9:], "want": list(range(8))}], "end": [short_id]}]
    got = H.replay(rp, steps, {short_id: reqs[short_id], long_id: reqs[long_id]})
    assert np.abs(got[short_id] - ref[short_id]).max() <= tolerance("float32", ref)


def test_pool_too_small_is_reported(setups):
    from kvcm_amd.engine.replay import ReplayError, TraceReplayer
    d, reqs, ref, _ = setups[("A", "float32")]
    rp = TraceReplayer(d, "float32", max_tokens=64, block_size=16)
    with pytest.raises(ReplayError, match="does not fit"):
        rp.step({"step": 0, "entries": [{"id": "x", "tokens": reqs["r5"], "want": [0]}], "end": []})
    assert rp.core.blocks_in_use() == 0
    rp.step({"step": 1, "entries": [{"id": "y", "tokens": reqs["r5"][:60], "want": [0]}], "end": []})
    with pytest.raises(ReplayError, match="out of cache pages"):
        rp.step({"step": 2, "entries": [{"id": "y", "tokens": reqs["r5"][60:70], "want": [0]}], "end": []})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(setups, dtype, tmp_path):
    """bin/trace_run as a user runs it: steps on standard input, <step>.f32 files, 'done <step>'."""
    d, reqs, ref, _ = setups[("A", dtype)]
    sub = {rid: reqs[rid] for rid in ("r1", "r2", "r3", "r6")}
    steps = H.schedule_mixed(sub, seed=5)
    out = tmp_path / "out"
    env = dict(os.environ, HOME=str(tmp_path))
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", str(H.tokens_needed(sub))],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       env=env, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:len(steps)] == [f"done {s['step']}" for s in steps]
    V = H.TINY_A["vocab_size"]
    got = {rid: np.full((len(t), V), np.nan, dtype=np.float32) for rid, t in sub.items()}
    pos = {rid: 0 for rid in sub}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = out / f"{s['step']}.f32"
        if not wanted:
            assert not path.exists()
            continue
        logits = np.fromfile(path, dtype="<f4").reshape(wanted, V)
        row = 0
        for e in s["entries"]:
            for w in e["want"]:
                got[e["id"]][pos[e["id"]] + w] = logits[row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
    bad = H.first_difference(got, {rid: ref[rid] for rid in sub}, tolerance(dtype, ref))
    assert bad is None, f"first wrong logits at request {bad[0]} position {bad[1]}: error {bad[2]:.3g}"


def test_trace_run_reports_bad_input_and_stops(setups, tmp_path):
    """A step the program cannot run ends it with one line on stderr and exit code 1; the steps
    before it are done."""
    d, reqs, ref, _ = setups[("A", "float32")]
    good = {"step": 0, "entries": [{"id": "a", "tokens": reqs["r0"], "want": [0]}], "end": []}
    for bad, message in (({"step": 1, "entries": [{"id": "a", "tokens": [10 ** 6], "want": []}], "end": []}, "outside the vocabulary"),
                         ({"step": 1, "entries": [], "end": ["nobody"]}, "not live"),
                         ({"step": 1, "entries": [{"id": "a", "tokens": [1, 2], "want": [5]}], "end": []}, "wanted place"),
                         ("not json", "line 2"), ({"entries": []}, "JSON object")):
        lines = [json.dumps(good), bad if isinstance(bad, str) else json.dumps(bad)]
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                            "--out", str(tmp_path / "o"), "--max-tokens", "128"], input="\n".join(lines) + "\n",
                           capture_output=True, text=True, env=dict(os.environ, HOME=str(tmp_path)), timeout=300)
        assert p.returncode == 1 and p.stdout.strip() == "done 0", (p.returncode, p.stdout, p.stderr[-500:])
        assert "trace_run: input line 2" in p.stderr and message in p.stderr, p.stderr[-500:]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_scheduled_program(setups, dtype, tmp_path):
    """bin/trace_run --scheduled: requests with given continuations go through the engine's own scheduler
    (portions of 16, a pool small enough that pages are used again, arrivals at different steps) and
    <id>.f32 holds the logits each given token was to be sampled from."""
    d, reqs, ref, _ = setups[("A", dtype)]
    names = ["r1", "r2", "r3", "r6", "r0"]
    lines, cut = [], {}
    for k, rid in enumerate(names):
        toks = reqs[rid]
        n = max(1, min(6, len(toks) - 1))
        cut[rid] = len(toks) - n
        lines.append(json.dumps({"id": rid, "prompt": toks[:cut[rid]], "forced": toks[cut[rid]:], "arrival": 2 * k}))
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--scheduled", "--model", d, "--dtype", dtype,
                        "--out", str(out), "--max-seq-len", "128", "--num-blocks", "12", "--max-num-seqs", "3",
                        "--prefill-chunk", "16", "--max-batched-tokens", "40", "--dump-tables"],
                       input="\n".join(lines) + "\n", capture_output=True, text=True,
                       env=dict(os.environ, HOME=str(tmp_path)), timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split() == [w for rid in names for w in ("done", rid)]
    V = H.TINY_A["vocab_size"]
    tol = tolerance(dtype, ref)
    for rid in names:
        toks = reqs[rid]
        got = np.fromfile(out / f"{rid}.f32", dtype="<f4").reshape(len(toks) - cut[rid], V)
        want = ref[rid][cut[rid] - 1:len(toks) - 1]
        err = np.abs(got.astype(np.float64) - want).max()
        assert err <= tol, f"request {rid}: error {err:.3g}"
    tables = json.loads((out / "0.tables.json").read_text())
    assert tables["step"] == 0 and [t["id"] for t in tables["tables"]] == ["r1"]
    # the plain replay writes the same kind of dump
    steps = H.schedule_whole({"r1": reqs["r1"]})
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "128", "--dump-tables"], input=json.dumps(steps[0]) + "\n", capture_output=True,
                       text=True, env=dict(os.environ, HOME=str(tmp_path)), timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    dump = json.loads((out / "0.tables.json").read_text())
    pages = -(-len(reqs["r1"]) // 16)
    assert dump["tables"][0]["id"] == "r1" and len(dump["tables"][0]["groups"][0]) == pages


@pytest.mark.parametrize("case", [("A", "float32"), ("B", "bfloat16"), ("D", "bfloat16"), ("D", "float32"), ("E", "bfloat16")])
def test_replay_through_recorded_step_programs(setups, case):
    """The same schedules with every step run the way generation runs it by default: from the launch list
    recorded at the first step of its shape, replayed with nothing but the step's metadata changed.  Every
    position's logits are fetched, so a value that a recording took from its own step instead of the
    metadata (a position, a page, a row count) shows at the first replay that differs in it."""
    from kvcm_amd.engine.replay import TraceReplayer
    d, reqs, ref, _ = setups[case]
    name, dtype = case
    rp = TraceReplayer(d, dtype, max_tokens=H.tokens_needed(reqs), block_size=H.BLOCK_SIZE[name], use_programs=True)
    assert rp.programs is not None
    for steps in (H.schedule_portions(reqs), H.schedule_mixed(reqs, seed=3), H.schedule_tail_singly(reqs, 32)):
        got = H.replay(rp, steps, reqs)
        assert all(not np.isnan(g).any() for g in got.values())
        bad = H.first_difference(got, ref, tolerance(dtype, ref))
        assert bad is None, f"first wrong logits at request {bad[0]} position {bad[1]}: error {bad[2]:.3g}"
        assert rp.core.blocks_in_use() == 0
    assert rp.steps_replayed > 3 * len(rp.programs) > 0, (rp.steps_replayed, len(rp.programs))
    shapes = set(rp.programs)
    assert any(s.max_run > 1 and s.seqs > 1 for s in shapes) and any(s.max_run == 1 for s in shapes)
