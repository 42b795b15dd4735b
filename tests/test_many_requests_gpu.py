"""Decode steps of many requests, by value: 20, 64 and 140 live requests through the engine's own
scheduler with their continuations forced, at the matrix-core sizes (configurations D and E) and at
the layer widths of a served model, in bfloat16 and in 32-bit, against the plain implementation.
These are the paths behind the throughput figures at batch 64 and beyond: decode graphs of 32 and
64 rows (products that share their rows through LDS and leave split-K sums, norms that add them up,
the SwiGLU epilogue, the one-launch attention, padding to a bucket) and decode steps of more than
128 rows, which replay a recorded program with the library's products."""
import numpy as np
import pytest
import torch

import helpers as H
import plain_llama as plain

pytestmark = pytest.mark.gpu

REAL = dict(architectures=["LlamaForCausalLM"], vocab_size=32000, hidden_size=2048, intermediate_size=5632,
            num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=4, head_dim=64,
            max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
LIVE = (20, 64, 140)


def _requests(raw, count, prompt_range, seed):
    """(prompt, continuation) pairs: prompts of lengths in ``prompt_range``, 6 to 10 given tokens each."""
    rng = np.random.default_rng(seed)
    V = raw["vocab_size"]
    return [(rng.integers(0, V, size=int(rng.integers(*prompt_range))).tolist(),
             rng.integers(0, V, size=int(rng.integers(6, 11))).tolist()) for _ in range(count)]


def _reference(pm, requests):
    """The plain implementation's logits at the places the given tokens are sampled from."""
    seqs = [p + c for p, c in requests]
    rows = [list(range(len(p) - 1, len(p) + len(c) - 1)) for p, c in requests]
    return pm.logits_of_many(seqs, rows)


def _tiny_setup(tmp_path_factory, name, dtype):
    raw = H.CONFIGS[name]
    d = str(tmp_path_factory.mktemp(f"many_{name}_{dtype}"))
    H.make_model_dir(d, raw, H.WEIGHT_SEED[name], torch.bfloat16 if dtype == "bfloat16" else torch.float32, sharpen=H.SHARPEN[name])
    pm = plain.load_model_dir(d, plain.round_bf16 if dtype == "bfloat16" else None)
    requests = _requests(raw, max(LIVE) + 12, (30, 301), seed=41 + H.WEIGHT_SEED[name])
    return dict(model_dir=d), requests, _reference(pm, requests), H.BLOCK_SIZE[name]


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    return {(n, dt): _tiny_setup(tmp_path_factory, n, dt) for n, dt in (("D", "bfloat16"), ("E", "bfloat16"), ("D", "float32"))}


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    from kvcm_amd.config.model_config import LlamaConfig
    from kvcm_amd.weights.random_init import random_tensors
    cfg = LlamaConfig.from_dict(REAL)
    tensors = random_tensors("LlamaForCausalLM", cfg, seed=23, dtype=torch.float32, std=0.02, norm_jitter=0.1, device="cuda:0")
    for name in tensors:          # as in the tiny configurations: scores spread over a few units, a residual stream of order one
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            tensors[name] *= 1.5
        if "embed_tokens" in name:
            tensors[name] *= 20.0
    # short prompts: the plain implementation runs every token of every request in float64 at these widths
    requests = _requests(REAL, max(LIVE) + 12, (4, 25), seed=43)
    out = {}
    for dtype in ("bfloat16", "float32"):
        stored = {k: v.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32) for k, v in tensors.items()}
        pm = plain.PlainLlama(REAL, {k: v.float().cpu().numpy() for k, v in stored.items()}, plain.round_bf16 if dtype == "bfloat16" else None)
        out[dtype] = (dict(architecture="LlamaForCausalLM", model_config=cfg, tensors=stored), requests, _reference(pm, requests), 16)
    return out


def _run(setup, dtype, live, tolerance):
    """``live`` + 12 requests through an engine that holds ``live`` at a time; the first step takes all the
    prompts that fit, so that they decode side by side.  Returns the engine after the comparison."""
    from kvcm_amd import Engine, EngineConfig
    from kvcm_amd.engine.replay import scheduled_replay
    source, requests, ref, B = setup
    requests, ref = requests[:live + 12], ref[:live + 12]
    tokens = sum(len(p) + len(c) for p, c in requests)
    longest = max(len(p) + len(c) for p, c in requests)
    ec = EngineConfig(block_size=B, num_blocks=sum(-(-(len(p) + len(c)) // B) for p, c in requests) + 8,
                      max_seq_len=-(-longest // 64) * 64, max_num_seqs=live, max_batched_tokens=-(-tokens // 64) * 64, dtype=dtype,
                      max_logit_rows=max(live, 64), beyond_max_position=True)
    eng = Engine(source.get("model_dir"), ec, **{k: v for k, v in source.items() if k != "model_dir"})
    ops = eng.runner.ops
    sums_added_by_norms = []
    real_rmsnorm = ops.rmsnorm

    def counting(x, weight, out, eps, add=None, rows=None, write_back=True):
        if isinstance(add, ops.PartialSums):
            sums_added_by_norms.append(x.shape[0])
        return real_rmsnorm(x, weight, out, eps, add=add, rows=rows, write_back=write_back)

    ops.rmsnorm = counting
    try:
        got = scheduled_replay(eng, requests, max_steps=2000)
    finally:
        ops.rmsnorm = real_rmsnorm
    scale = max(1.0, max(float(np.abs(r).max()) for r in ref))
    worst = 0.0
    for i, (g, r) in enumerate(zip(got, ref)):
        assert not np.isnan(g).any(), (live, i, "a forced token has no logits")
        err = np.abs(g - r).max(axis=1)
        worst = max(worst, float(err.max()))
        bad = np.nonzero(err > tolerance * scale)[0]
        assert len(bad) == 0, (f"{live} live: request {i} (prompt {len(requests[i][0])}), given token {bad[0]}: "
                               f"error {err[bad[0]]:.3g} > {tolerance * scale:.3g}")
    print(f"{dtype} {live} live: largest error {worst:.3g} of {tolerance * scale:.3g}")
    assert eng.core.blocks_in_use() == 0 and eng.core.counters()["max_running"] == live
    eng.sums_added_by_norms = sums_added_by_norms
    return eng


def _decode_shapes(eng):
    return {(s.rows, kind) for s, kind in eng.recorded.recorded_shapes.items() if s.max_run == 1}


def _check_paths(eng, live, dtype, products_split=False):
    """The step shapes the run was meant to go through were recorded and replayed."""
    shapes = _decode_shapes(eng)
    st = eng.recorded.stats()
    assert st["steps_replayed"] > 0
    if live == 20:
        assert (20, "graph") in shapes, shapes           # the bucket of 32 rows, cut down to this engine's 20 sequences
    elif live == 64:
        assert (64, "graph") in shapes, shapes
    else:
        assert (140, "program") in shapes, shapes        # more than 128 rows: a program with the library's products
        assert any(rows in (96, 128) and kind == "graph" for rows, kind in shapes), shapes      # as requests finish
    assert st["steps_as_graph"] > 0
    if products_split and dtype == "bfloat16" and live in (20, 64):
        # split-K sums went from the products to the norms un-added (recorded once per shape, then replayed);
        # at the tiny widths a product of these rows is not split
        assert any(rows >= 17 for rows in eng.sums_added_by_norms), eng.sums_added_by_norms


@pytest.mark.parametrize("live", LIVE)
@pytest.mark.parametrize("case", [("D", "bfloat16"), ("E", "bfloat16"), ("D", "float32")], ids=lambda c: f"{c[0]}-{c[1]}")
def test_many_live_requests_at_matrix_core_sizes(tiny, case, live):
    dtype = case[1]
    eng = _run(tiny[case], dtype, live, 1e-2 if dtype == "bfloat16" else 1e-5)
    _check_paths(eng, live, dtype)


@pytest.mark.parametrize("live", LIVE)
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_many_live_requests_at_real_widths(real, dtype, live):
    eng = _run(real[dtype], dtype, live, 1e-2 if dtype == "bfloat16" else 1e-4)
    _check_paths(eng, live, dtype, products_split=True)
