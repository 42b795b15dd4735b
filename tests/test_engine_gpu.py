"""The engine as a user meets it: generation through the entry point (greedy and with a
temperature), the scheduler under page pressure with real logits, prefix caching, paged against
contiguous, graphs against eager steps, and each part of a layer on its own."""
import math

import numpy as np
import pytest
import torch

import helpers as H
import plain_llama as plain

pytestmark = pytest.mark.gpu


def _engine(d, **kw):
    from kvcm_amd import Engine, EngineConfig
    base = dict(block_size=16, num_blocks=64, max_seq_len=256, max_num_seqs=8, max_batched_tokens=256, dtype="float32")
    base.update(kw)
    if base.get("use_graphs") is False:            # "no graphs" in these tests means: every step launch by launch
        base.setdefault("use_programs", False)
    return Engine(d, EngineConfig(**base))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in ("A", "B"):
        for dtype in ("float32", "bfloat16"):
            d = str(tmp_path_factory.mktemp(f"gen_{name}_{dtype}"))
            H.make_model_dir(d, H.CONFIGS[name], H.WEIGHT_SEED[name], torch.float32 if dtype == "float32" else torch.bfloat16)
            out[(name, dtype)] = (d, plain.load_model_dir(d, plain.round_bf16 if dtype == "bfloat16" else None))
    return out


def _prompts(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, raw["vocab_size"], size=n).tolist() for n in lengths]


def _same_up_to_near_ties(got, want, margins, tie):
    """Token lists agree; the first difference, if any, sits where the plain model's two best
    scores are closer than ``tie`` (after it the continuations legitimately differ)."""
    for k, (g, w) in enumerate(zip(got, want)):
        if g != w:
            return margins[k] < tie
    return len(got) == len(want)


# ------------------------------------------------------------------------------ generation
def _serve_natively(eng, prompts, new_tokens, first_id):
    """Serves the prompts through the native engine object alone (csrc/hip/kvcm_hip.h: kvcm_engine_add /
    step / idle / take_finished), as a C caller would; the interpreter is entered only for a step whose
    shape has no program yet.  -> (generated ids per prompt, steps run natively, steps recorded)."""
    import ctypes as C
    lib, h = eng.runner.ops.lib(), eng.recorded.native_handle
    for k, p in enumerate(prompts):
        arr = (C.c_int32 * len(p))(*p)
        assert lib.kvcm_engine_add(h, first_id + k, arr, len(p), new_tokens, 0.0, 0, eng.now()) == 0
    info, native, recorded, out = (C.c_int64 * 8)(), 0, 0, {}
    for _ in range(10000):
        if lib.kvcm_engine_idle(h):
            break
        rc = lib.kvcm_engine_step(h, eng.now(), info)
        assert rc >= 0, lib.kvcm_hip_last_error().decode()
        if rc == 1:
            native += 1
        elif rc == 0:                       # a shape the engine has not met: the parts run it once, recording
            eng.step(planned_natively=True)
            recorded += 1
        n = lib.kvcm_engine_take_finished(h)
        meta, times = (C.c_int64 * 6)(), (C.c_double * 4)()
        for i in range(n):
            size = lib.kvcm_engine_finished_get(h, i, meta, times, None, 0)
            toks = (C.c_int32 * size)()
            assert lib.kvcm_engine_finished_get(h, i, meta, times, toks, size) == size
            out[int(meta[0])] = list(toks)[int(meta[1]):]
        lib.kvcm_engine_finished_clear(h)
    assert lib.kvcm_engine_idle(h)
    return [out[first_id + k] for k in range(len(prompts))], native, recorded


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_native_caller_serves_through_the_engine_object(models, dtype):
    """Requests in, steps, finished requests out through the C entry points alone: once the step shapes of a
    workload are recorded no step enters the interpreter, and the tokens are those of the Python engine; a
    workload with shapes not met before falls back to recording, step by step, and goes on natively."""
    d, pm = models[("A", dtype)]
    prompts = _prompts(H.TINY_A, [7, 13, 5, 30], seed=21)
    eng = _engine(d, dtype=dtype)
    want = eng.generate(prompts, max_new_tokens=9)              # records the shapes this workload meets
    got, native, recorded = _serve_natively(eng, prompts, 9, first_id=100)
    assert got == want
    assert recorded == 0 and native >= 9, (native, recorded)
    assert eng.core.blocks_in_use() == 0
    # other prompt lengths and another number of requests: new shapes turn up mid-run
    others = _prompts(H.TINY_A, [40, 3, 3, 19, 8, 11], seed=22)
    got, native, recorded = _serve_natively(eng, others, 6, first_id=200)
    assert recorded >= 1 and native >= 1, (native, recorded)
    fresh = _engine(d, dtype=dtype, use_graphs=False).generate(others, max_new_tokens=6)
    assert got == fresh
    assert eng.core.blocks_in_use() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_config_a(models, dtype):
    """Tiny A: three requests with prompts of 7, 13 and 5 ids, 8 greedy tokens each."""
    d, pm = models[("A", dtype)]
    prompts = _prompts(H.TINY_A, [7, 13, 5], seed=1)
    eng = _engine(d, dtype=dtype)
    got = eng.generate(prompts, max_new_tokens=8)
    for p, g in zip(prompts, got):
        want, margins = pm.generate(p, 8)
        assert _same_up_to_near_ties(g, want, margins, 1e-4 if dtype == "float32" else 5e-2), (g, want, margins)
    assert eng.core.blocks_in_use() == 0 and eng.idle()
    solo = [_engine(d, dtype=dtype, use_graphs=False).generate([p], 8)[0] for p in prompts]
    assert solo == got, "a request's tokens changed with the batch it ran in"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_generation_config_b_chunked(models, dtype):
    """Tiny B: prompts of 1, 9, 17, 33 and 40 ids, prefill in portions of 16 mixed with decodes,
    12 tokens each at temperature 0.8 under a fixed sampler seed."""
    d, pm = models[("B", dtype)]
    prompts = _prompts(H.TINY_B, [1, 9, 17, 33, 40], seed=3)
    eng = _engine(d, dtype=dtype, block_size=8, num_blocks=40, prefill_chunk=16, max_batched_tokens=24)
    ids = [eng.add_request(p, 12, temperature=0.8, seed=1234) for p in prompts]
    mixed = 0
    done = {}
    while not eng.idle():
        plan_before = eng.core.num_running()
        info = eng.step()
        mixed += info.prefill_tokens > 0 and info.decode_seqs > 0
        for f in eng.take_finished():
            done[f.id] = f.generated
    assert mixed > 0, "no step mixed a prompt portion with decoded tokens"
    for rid, p in zip(ids, prompts):
        want, margins = pm.generate(p, 12, temperature=0.8, seed=1234, request_id=rid)
        assert _same_up_to_near_ties(done[rid], want, margins, 1e-4 if dtype == "float32" else 5e-2), (done[rid], want)
    # the same requests, whole prompts, other batch order: the draw depends on (seed, request, index) only
    eng2 = _engine(d, dtype=dtype, block_size=8, num_blocks=40)
    for rid, p in reversed(list(zip(ids, prompts))):
        eng2.add_request(p, 12, temperature=0.8, seed=1234, request_id=rid)
    again = {f.id: f.generated for f in eng2.run_until_idle()}
    if dtype == "float32":
        assert again == done


# wide enough (K = 1024) that the QKV product of a step of about a hundred rows splits K: the mixed
# step then starts from partial sums
TINY_WIDE = dict(architectures=["LlamaForCausalLM"], vocab_size=300, hidden_size=1024, intermediate_size=1408,
                 num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2, head_dim=64,
                 max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)


@pytest.mark.parametrize("raw,chunk,budget,sharpen", [(H.TINY_D, 160, 200, H.SHARPEN["D"]), (TINY_WIDE, 100, 110, 3.0)],
                         ids=["narrow", "wide_split_k"])
def test_mixed_steps_at_matrix_core_sizes(tmp_path, raw, chunk, budget, sharpen):
    """head_dim 64, bfloat16: decoding requests (the scheduler puts them first) take the one-launch
    decode kernel inside steps that also carry long prompt portions for the tiled kernel; graphs
    replay the pure decode steps.  Greedy tokens must be those of the plain implementation."""
    d = str(tmp_path / "m")
    H.make_model_dir(d, raw, H.WEIGHT_SEED["D"], torch.bfloat16, sharpen=sharpen)
    pm = plain.load_model_dir(d, plain.round_bf16)
    prompts = _prompts(raw, [40, 12, 700, 90, 1200, 25], seed=9)
    # (steps launch by launch, so that the kernels each step takes can be counted here; recorded steps
    # have a test of their own below)
    eng = _engine(d, dtype="bfloat16", num_blocks=200, max_seq_len=2048, prefill_chunk=chunk, max_batched_tokens=budget,
                  use_programs=False)
    ids = [eng.add_request(p, 10) for p in prompts]
    qkv_width = (raw["num_attention_heads"] + 2 * raw["num_key_value_heads"]) * raw["head_dim"]
    split_seen = False
    # which attention kernels the steps take (a silent fall back to the general kernel would pass the comparison)
    ops, calls = eng.runner.ops, {"fused": 0, "fused_in_mixed": 0, "tiled": 0, "general": 0}
    real = (ops.attention_decode_fused, ops.attention_prefill, ops.attention)

    def fused(*a, **k):
        calls["fused"] += 1
        return real[0](*a, **k)

    def tiled(*a, **k):
        calls["tiled"] += 1
        return real[1](*a, **k)

    def general(*a, **k):
        calls["general"] += 1
        return real[2](*a, **k)

    ops.attention_decode_fused, ops.attention_prefill, ops.attention = fused, tiled, general
    try:
        mixed_big, done = 0, {}
        while not eng.idle():
            before = dict(calls)
            info = eng.step()
            # (a plan is in admission order: where an older request still runs its prompt while a
            # younger one decodes, no decode row leads and the tiled kernel takes them all)
            if info.decode_seqs > 0 and info.prefill_tokens >= chunk - 60 and eng.core.plan_leading > 0:
                mixed_big += 1
                split_seen |= ops.skinny_splits(info.rows, qkv_width, raw["hidden_size"]) > 1
                calls["fused_in_mixed"] += calls["fused"] > before["fused"] and calls["tiled"] > before["tiled"]
            for f in eng.take_finished():
                done[f.id] = f.generated
    finally:
        ops.attention_decode_fused, ops.attention_prefill, ops.attention = real
    assert mixed_big > 3, "no step mixed decoding requests with a long prompt portion"
    assert calls["fused_in_mixed"] == mixed_big and calls["general"] == 0, calls
    assert split_seen == (raw is TINY_WIDE)
    for rid, p in zip(ids, prompts):
        want, margins = pm.generate(p, 10)
        assert _same_up_to_near_ties(done[rid], want, margins, 5e-2), (rid, done[rid], want, margins)
    assert eng.core.blocks_in_use() == 0


def test_preemption_recomputes_and_gives_the_same_tokens(models):
    d, pm = models[("A", "float32")]
    prompts = _prompts(H.TINY_A, [20, 25, 18, 30, 22, 19], seed=5)
    roomy = _engine(d, num_blocks=64).generate(prompts, 24)
    tight = _engine(d, num_blocks=9, watermark_blocks=0)       # 144 slots for 6 x (about 45) tokens
    got = tight.generate(prompts, 24)
    assert tight.core.counters()["preemptions"] > 0
    assert got == roomy
    assert tight.core.blocks_in_use() == 0


def test_impossible_request_is_rejected_and_the_rest_served(models):
    d, pm = models[("A", "float32")]
    eng = _engine(d, num_blocks=4)
    prompts = _prompts(H.TINY_A, [100, 10], seed=6)
    out = eng.generate(prompts, 4)
    assert out[0] == [] and len(out[1]) == 4 and eng.core.counters()["rejected"] == 1


def test_paged_equals_contiguous_and_prefix_cache_changes_nothing(models):
    d, pm = models[("B", "float32")]
    rng = np.random.default_rng(7)
    shared = rng.integers(0, 384, size=40).tolist()
    prompts = [shared + rng.integers(0, 384, size=n).tolist() for n in (5, 9, 3)]
    base = [_engine(d, block_size=8, num_blocks=64).generate([p], 10)[0] for p in prompts]
    contiguous = _engine(d, block_size=8, num_blocks=128, policy="contiguous", max_seq_len=128)
    assert [contiguous.generate([p], 10)[0] for p in prompts] == base
    cached = _engine(d, block_size=8, num_blocks=64, prefix_caching=True)
    got = [cached.generate([p], 10)[0] for p in prompts]
    st = cached.core.prefix_stats()
    assert st["hit_blocks"] >= 2 * 5 and cached.core.counters()["prefill_tokens_saved"] >= 80
    assert got == base
    assert cached.generate([prompts[0]], 10)[0] == base[0]        # a full re-run hits its own pages
    with pytest.raises(RuntimeError, match="prefix caching"):
        cached.score(prompts[0])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_score_gives_teacher_forced_logits(models, dtype):
    d, pm = models[("A", dtype)]
    toks = _prompts(H.TINY_A, [90], seed=8)[0]
    eng = _engine(d, dtype=dtype)
    got = eng.score(toks)
    ref = pm.logits(toks)
    tol = (1e-5 if dtype == "float32" else 1e-2) * max(1.0, np.abs(ref).max())
    assert np.abs(got - ref).max() <= tol
    assert eng.core.blocks_in_use() == 0


def test_limits_and_bad_tokens_are_refused(models):
    d, _ = models[("A", "float32")]
    eng = _engine(d)
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([1, 2, 256], 4)
    with pytest.raises(ValueError, match="at least one token"):
        eng.add_request([], 4)
    small = _engine(d, max_batched_tokens=16, max_num_seqs=2, max_seq_len=64)
    with pytest.raises(RuntimeError, match="exceeds model limits"):
        small.runner.run_entries([])  # nothing to run is fine ...
        small.core.seq_new(99, list(range(100)))
        small.core.admit(99)
        small.runner.run_entries([(99, 0, 100, None)])            # ... more rows than the buffers hold is not


# ---------------------------------------------------------------------------------- graphs
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(models, dtype):
    """Decode steps replayed from a captured graph, several times with eager work and
    synchronisations in between, give the tokens of eager decoding."""
    d, pm = models[("A", dtype)]
    prompts = _prompts(H.TINY_A, [9, 30, 4, 17, 12], seed=9)
    eager = _engine(d, dtype=dtype, use_graphs=False).generate(prompts, 20)
    eng = _engine(d, dtype=dtype, use_graphs=True)
    ids = [eng.add_request(p, 20) for p in prompts[:3]]
    done = {}
    step = 0
    while not eng.idle():
        eng.step()
        step += 1
        if step == 4:                                             # eager work between replays: new prompts arrive
            ids += [eng.add_request(p, 20) for p in prompts[3:]]
        if step % 5 == 0:
            eng.score(prompts[1])                                 # an eager step through the same buffers
            torch.cuda.synchronize()
        for f in eng.take_finished():
            done[f.id] = f.generated
    assert eng.decode_graphs.graph_shapes(), "no graph was captured"
    assert [done[i] for i in ids] == eager


def test_graph_replays_at_matrix_core_sizes(tmp_path):
    """head_dim 64, bfloat16: replayed decode steps (split products whose sums the one-launch decode
    kernel and the norms add up, batch padded to a bucket, launch sized for the longest context
    allowed) give the plain implementation's tokens, also while contexts cross chunks of 256."""
    d = str(tmp_path / "m")
    H.make_model_dir(d, H.TINY_D, H.WEIGHT_SEED["D"], torch.bfloat16, sharpen=H.SHARPEN["D"])
    pm = plain.load_model_dir(d, plain.round_bf16)
    prompts = _prompts(H.TINY_D, [250, 20, 505, 65, 1019], seed=11)
    eng = _engine(d, dtype="bfloat16", num_blocks=200, max_seq_len=2048, max_batched_tokens=2048, use_graphs=True)
    got = eng.generate(prompts, 24)
    assert eng.decode_graphs.graph_shapes(), "no graph was captured"
    for p, g in zip(prompts, got):
        want, margins = pm.generate(p, 24)
        assert _same_up_to_near_ties(g, want, margins, 5e-2), (len(p), g, want, margins)
    eager = _engine(d, dtype="bfloat16", num_blocks=200, max_seq_len=2048, max_batched_tokens=2048, use_graphs=False)
    assert eager.generate(prompts, 24) == got


def test_graphs_follow_the_context_across_classes(tmp_path):
    """An engine that allows 4,096 tokens captures decode graphs per context class (1,024, 2,048,
    4,096): each replays the decode attention with the parts that suit its bound.  A request that
    crosses 2,048 while decoding changes class on the way."""
    d = str(tmp_path / "m")
    H.make_model_dir(d, H.TINY_D, H.WEIGHT_SEED["D"], torch.bfloat16, sharpen=H.SHARPEN["D"])
    pm = plain.load_model_dir(d, plain.round_bf16)
    prompts = _prompts(H.TINY_D, [2030, 100], seed=13)
    # (the tiny model states 2,048 positions; running past them is what this test is about)
    kw = dict(dtype="bfloat16", num_blocks=300, max_seq_len=4096, max_batched_tokens=4096, beyond_max_position=True)
    eng = _engine(d, use_graphs=True, **kw)
    got = eng.generate(prompts, 40)
    assert eng.decode_graphs.graph_shapes() == [(2, 2048), (2, 4096)]
    assert _engine(d, use_graphs=False, **kw).generate(prompts, 40) == got
    for p, g in zip(prompts, got):
        want, margins = pm.generate(p, 40)
        assert _same_up_to_near_ties(g, want, margins, 5e-2), (len(p), g, want, margins)


@pytest.mark.parametrize("attn", ["v1", "v2"])
def test_attention_variants_at_matrix_core_sizes(tmp_path, attn):
    """--attn v1 (one-pass kernel everywhere) and v2 (partitions + merge for decode steps, after a
    separate rotation + page write that reads the split sums) give the plain implementation's
    tokens too; "auto" is covered by the tests above."""
    d = str(tmp_path / "m")
    H.make_model_dir(d, H.TINY_D, H.WEIGHT_SEED["D"], torch.bfloat16, sharpen=H.SHARPEN["D"])
    pm = plain.load_model_dir(d, plain.round_bf16)
    prompts = _prompts(H.TINY_D, [250, 33, 520], seed=12)
    eng = _engine(d, dtype="bfloat16", num_blocks=100, max_seq_len=1024, max_batched_tokens=1024, attn=attn)
    ops, calls = eng.runner.ops, {"fused": 0, "partitioned": 0}
    real = (ops.attention_decode_fused, ops.attention_decode)

    def fused(*a, **k):
        calls["fused"] += 1
        return real[0](*a, **k)

    def partitioned(*a, **k):
        calls["partitioned"] += 1
        return real[1](*a, **k)

    ops.attention_decode_fused, ops.attention_decode = fused, partitioned
    try:
        got = eng.generate(prompts, 12)
    finally:
        ops.attention_decode_fused, ops.attention_decode = real
    assert calls["fused"] == 0 and (calls["partitioned"] > 0) == (attn == "v2"), calls
    for p, g in zip(prompts, got):
        want, margins = pm.generate(p, 12)
        assert _same_up_to_near_ties(g, want, margins, 5e-2), (len(p), g, want, margins)


# -------------------------------------------------------------------------- parts, alone
def _ctx(dtype, hidden):
    from kvcm_amd import ops
    from kvcm_amd.parts.base import BuildContext
    return BuildContext(dtype, torch.device("cuda:0"), hidden, 8, ops)


def _step_base():
    from kvcm_amd.parts.base import StepView
    return StepView


class _Step(_step_base()):
    """The little of a step that a part needs when it is run on its own: the declared view of a step
    (parts.base.StepView) with the arrays this part reads."""

    def __init__(self, rows, positions=None):
        self.rows = self.real_rows = rows
        self.positions = None if positions is None else torch.tensor(positions, dtype=torch.int32, device="cuda:0")
        self.tokens = None
        self._bufs = {}

    def ws(self, name, shape, dtype=None):
        key = (name, tuple(shape), dtype)
        if key not in self._bufs:
            self._bufs[key] = torch.zeros(*shape, dtype=dtype or self.default, device="cuda:0")
        return self._bufs[key]


def _dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device="cuda:0")


def test_part_rmsnorm_alone():
    from kvcm_amd.registry import NORMS
    rng = np.random.default_rng(20)
    H_, T = 200, 5
    part = NORMS.get("rmsnorm")({"size": H_, "eps": 3e-6}, "n.", _ctx(torch.float32, H_))
    w = rng.normal(size=H_)
    part.bind({"weight": _dev(w)})
    x = rng.normal(size=(T, H_)).astype(np.float32)
    out = torch.zeros(T, H_, device="cuda:0")
    part.forward(_dev(x), out)
    np.testing.assert_allclose(out.cpu().numpy(), plain.rms_norm(x, w, 3e-6), rtol=3e-6, atol=1e-6)
    assert [s.sources[0][0] for s in part.param_specs()] == ["n.weight"]


def test_part_rotary_alone():
    from kvcm_amd.registry import POSITIONS
    rng = np.random.default_rng(21)
    nh, nkv, hd, T = 3, 1, 24, 4
    part = POSITIONS.get("rotary")({"theta": 77777.0, "dim": hd}, "", _ctx(torch.float32, 64))
    qkv = rng.normal(size=(T, (nh + 2 * nkv) * hd)).astype(np.float32)
    pos = [0, 3, 50, 51]
    t = _dev(qkv)
    step = _Step(T, pos)
    assert part.apply(step, t, nh, nkv, hd) is False              # nothing stored without a cache
    got = t.cpu().numpy().reshape(T, nh + 2 * nkv, hd)
    ref = plain.rotary(qkv.reshape(T, nh + 2 * nkv, hd)[:, :nh + nkv], pos, 77777.0)
    np.testing.assert_allclose(got[:, :nh + nkv], ref, atol=2e-6)
    np.testing.assert_array_equal(got[:, nh + nkv:], qkv.reshape(T, -1, hd)[:, nh + nkv:])


def test_part_swiglu_alone():
    from kvcm_amd.registry import FEED_FORWARDS
    rng = np.random.default_rng(22)
    H_, I, T = 40, 72, 6
    part = FEED_FORWARDS.get("swiglu")({"intermediate_size": I}, "mlp.", _ctx(torch.float32, H_))
    wg, wu, wd = rng.normal(size=(I, H_)), rng.normal(size=(I, H_)), rng.normal(size=(H_, I))
    part.bind({"w_gate_up": _dev(np.concatenate([wg, wu])), "w_down": _dev(wd)})
    h = rng.normal(size=(T, H_)).astype(np.float32) * 0.3
    step = _Step(T)
    step.default = torch.float32
    out = part.forward(step, _dev(h))
    gu = np.concatenate([plain.linear(h, wg), plain.linear(h, wu)], axis=-1)
    np.testing.assert_allclose(out.cpu().numpy(), plain.linear(plain.swiglu(gu), wd), rtol=1e-4, atol=1e-4)
    names = [n for s in part.param_specs() for n, _ in s.sources]
    assert names == ["mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight"]


def test_part_attention_mixer_alone_through_the_cache():
    """The mixer on its own: one expert of everything else is the identity.  A prompt portion,
    then single tokens, against plain attention over the whole sequence."""
    from kvcm_amd.cache.storage import KVStorage
    from kvcm_amd.parts.base import KVCacheNeed, PartSpec
    from kvcm_amd.registry import MIXERS
    rng = np.random.default_rng(23)
    Hh, nh, nkv, hd, B, n = 48, 4, 2, 16, 8, 21
    ctx = _ctx(torch.float32, Hh)
    part = MIXERS.get("gqa_attention")({"num_heads": nh, "num_kv_heads": nkv, "head_dim": hd, "scale": 0.3, "window": 0,
                                       "position": PartSpec("rotary", {"theta": 1e4, "dim": hd})}, "a.", ctx)
    wq, wk, wv, wo = (rng.normal(size=s) * 0.3 for s in ((nh * hd, Hh), (nkv * hd, Hh), (nkv * hd, Hh), (Hh, nh * hd)))
    part.bind({"wqkv": _dev(np.concatenate([wq, wk, wv])), "wo": _dev(wo)})
    assert part.cache_need() == KVCacheNeed(nkv, hd, 0)
    store = KVStorage(0, part.cache_need(), 1, 6, B, torch.float32, "cuda:0")
    part.attach_cache(store, 0)
    h = rng.normal(size=(n, Hh)).astype(np.float32)
    table = [4, 1, 5]                                             # scattered pages

    class Step(_Step):
        default = torch.float32

        def __init__(self, lo, hi):
            super().__init__(hi - lo, list(range(lo, hi)))
            self.lo, self.hi = lo, hi

            self.max_run, self.real_seqs, self.seqs = hi - lo, 1, 1
            self.row_seq = _dev([0] * self.rows, torch.int32)
            self.ctx_lens = _dev([p + 1 for p in range(lo, hi)], torch.int32)
            self.max_context = self.max_context_bound = hi

        def slots(self, g):
            return _dev([table[p // B] * B + p % B for p in range(self.lo, self.hi)], torch.int32)

        def tables(self, g):
            return _dev(table, torch.int32)

        def table_stride(self, g):
            return 3

    outs = []
    for lo, hi in [(0, 13), (13, 14), (14, 19), (19, 20), (20, 21)]:
        outs.append(part.forward(Step(lo, hi), _dev(h[lo:hi])).cpu().numpy().copy())
    got = np.concatenate(outs)
    pos = np.arange(n)
    q = plain.rotary(plain.linear(h, wq).reshape(n, nh, hd), pos, 1e4)
    k = plain.rotary(plain.linear(h, wk).reshape(n, nkv, hd), pos, 1e4)
    v = plain.linear(h, wv).reshape(n, nkv, hd)
    ref = plain.linear(plain.attention(q, k, v, pos, pos, 0.3).reshape(n, nh * hd), wo)
    np.testing.assert_allclose(got, ref, atol=2e-4, rtol=1e-4)


def test_block_arrangement_alone():
    """pre-norm residual with stand-in parts: x + mixer(norm(x)) then + ffn(norm(.)), the last
    addition left pending."""
    from kvcm_amd.registry import BLOCKS
    from kvcm_amd.parts.base import FeedForward, Mixer, Norm

    class Twice(Norm):
        def forward(self, x, out, add=None, rows=None):
            if add is not None:
                x += add
            out.copy_(2 * x)
            return out

    class PlusOne(Mixer):
        def forward(self, step, h):
            return h + 1

    class Negate(FeedForward):
        def forward(self, step, h):
            return -h

    ctx = _ctx(torch.float32, 4)
    block = BLOCKS.get("prenorm_residual")({"norm_mixer": Twice({}, "", ctx), "mixer": PlusOne({}, "", ctx),
                                            "norm_ffn": Twice({}, "", ctx), "ffn": Negate({}, "", ctx)})
    step = _Step(2)
    step.default = torch.float32
    x = torch.ones(2, 4, device="cuda:0")
    pending = block.forward(step, x, torch.full((2, 4), 0.5, device="cuda:0"))
    # x = 1 + 0.5 = 1.5; mixer(2x) = 4; x = 5.5; ffn(2x) = -11 pending
    assert torch.equal(x, torch.full((2, 4), 5.5, device="cuda:0"))
    assert torch.equal(pending, torch.full((2, 4), -11.0, device="cuda:0"))


@pytest.mark.parametrize("which,dtype", [("D", "bfloat16"), ("E", "bfloat16"), ("D", "float32"), ("E", "float32")])
def test_random_workloads_over_engine_options(tmp_path, which, dtype):
    """Requests of random lengths arriving while others run, at the matrix-core sizes, over chunked and
    whole prompts, small and large budgets, prefix cache, recorded steps (programs, graphs) and a pool
    small enough to preempt, driven through the real scheduler with their continuations forced: the
    logits every token would have been sampled from equal the plain implementation's, every request
    ends with the number of tokens it asked for and every page comes back."""
    import itertools
    from kvcm_amd.engine.replay import scheduled_replay
    raw, B = H.CONFIGS[which], H.BLOCK_SIZE[which]
    d = str(tmp_path / "m")
    H.make_model_dir(d, raw, H.WEIGHT_SEED[which], torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                     sharpen=H.SHARPEN[which])
    pm = plain.load_model_dir(d, plain.round_bf16 if dtype == "bfloat16" else None)
    rng = np.random.default_rng(31)
    V = raw["vocab_size"]
    shared = rng.integers(0, V, size=100).tolist()
    requests = []
    for i, n in enumerate([1, 2, 16, 17, 60, 130, 257, 400, 700, 33, 64, 129, 5, 300]):
        toks = rng.integers(0, V, size=n).tolist()
        if i % 2:
            toks = (shared + toks)[:900]                       # every other request begins with the same 100 tokens
        requests.append((toks, rng.integers(0, V, size=int(rng.integers(1, 30))).tolist()))
    ref = []
    for prompt, cont in requests:
        ref.append(pm.logits(prompt + cont)[len(prompt) - 1:len(prompt) + len(cont) - 1])
    scale = max(1.0, max(float(np.abs(r).max()) for r in ref))
    tol = (1e-2 if dtype == "bfloat16" else 1e-5) * scale
    arrivals = [3 * i for i in range(len(requests))]
    preempted = replayed = graphs = 0
    combos = itertools.product((0, 37), (96, 512), (False, True), (True, False))
    for combo, (chunk, budget, prefix, recorded) in enumerate(combos):
        if dtype == "float32" and (combo % 3):                 # 32-bit: a third of the combinations
            continue
        eng = _engine(d, dtype=dtype, block_size=B, num_blocks=70 * 16 // B, max_seq_len=1024, max_num_seqs=8,
                      max_batched_tokens=budget, prefill_chunk=chunk, prefix_caching=prefix, use_graphs=recorded,
                      use_programs=recorded, beyond_max_position=True)      # (configuration E states 512 positions)
        got = scheduled_replay(eng, requests, arrivals, max_steps=5000)
        for i, (g, r) in enumerate(zip(got, ref)):
            assert not np.isnan(g).any(), (combo, i, "a forced token has no logits")
            err = np.abs(g - r).max(axis=1)
            bad = np.nonzero(err > tol)[0]
            assert len(bad) == 0, (f"options chunk={chunk} budget={budget} prefix={prefix} recorded={recorded}: request {i} "
                                   f"(prompt {len(requests[i][0])}), generated token {bad[0]}: error {err[bad[0]]:.3g} > {tol:.3g}")
        assert eng.core.blocks_in_use() == 0
        preempted += eng.core.counters()["preemptions"]
        if recorded:
            st = eng.recorded.stats()
            replayed += st["steps_replayed"]
            graphs += st["steps_as_graph"]
    assert preempted > 0, "the pool was meant to be small enough to preempt"
    assert replayed > 0 and graphs > 0, "no step was replayed from a recorded program or graph"
