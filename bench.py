"""Decode and prefill throughput of the engine at TinyLlama-1.1B sizes with random weights.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--prompt-len 512] [--layers L]
                  [--sizes tinyllama-1.1b|llama-2-7b|llama-3-8b] [--context-limit 2048] [--prefill-tokens 2048]
                  [--tune-products off|heuristic|all] [--no-points] [--only-prefill]

A "step" is one decode step of the whole engine (schedule, batch metadata, upload, model step on
the GPU, sampling, download, update).  W untimed steps, then exactly K timed steps between two
device synchronisations.  One JSON line is printed: decoded tokens a second at the default batch,
the same at batch 1 and 64, a 2,048-token prefill, and the decode step's memory roofline.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

# TinyLlama-1.1B sizes: 22 layers of width 2048, 32 query heads and 4 key/value heads of 64, SwiGLU width
# 5632, vocabulary 32000, context 2048
SIZES = dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
             num_attention_heads=32, num_key_value_heads=4, head_dim=64, max_position_embeddings=2048,
             rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)


def build_engine(cfg, dtype, max_num_seqs, max_batched_tokens, tensors, context_limit=2048, tune_products="off"):
    from kvcm_amd.config.engine_config import EngineConfig
    from kvcm_amd.engine.engine import Engine
    ec = EngineConfig(block_size=16, max_seq_len=context_limit, num_blocks=max_num_seqs * context_limit // 16,
                      max_num_seqs=max_num_seqs, max_batched_tokens=max_batched_tokens, dtype=dtype,
                      max_logit_rows=max(max_num_seqs, 64), tune_products=tune_products,
                      # random weights rotate any position: a context limit beyond the sizes' own is allowed
                      beyond_max_position=context_limit > cfg.max_position_embeddings)
    return Engine(config=ec, architecture="LlamaForCausalLM", model_config=cfg, tensors=tensors)


def prompt_step_count(batch, prompt_len, budget=4096):
    """Steps that the prompts of a batch take at most: whole prompts, as many a step as the token budget
    holds beside the tokens of the requests that decode already."""
    per_step = max(1, (budget - batch) // prompt_len)
    return -(-batch // per_step) + 2


def decode_run(eng, batch, prompt_len, steps, warmup, vocab, seed=1):
    """-> (seconds for `steps` decode steps, mean context length during them)."""
    import numpy as np
    import torch
    rng = np.random.default_rng(seed)
    # requests admitted first decode while the others' prompts still run: room for those steps too
    prompt_steps = prompt_step_count(batch, prompt_len, eng.config.max_batched_tokens)
    for _ in range(batch):
        eng.add_request(rng.integers(3, vocab, size=prompt_len).tolist(), max_new_tokens=warmup + steps + 24 + prompt_steps)
    extra = 0
    while True:                                 # prompts, whole, as many per step as the budget takes
        info = eng.step()
        if info.prefill_tokens == 0 and eng.core.num_waiting() == 0:
            break
        extra += 1
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        info = eng.step()
        assert info.decode_seqs == batch and info.prefill_tokens == 0, "a timed step was not a pure decode step"
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx = prompt_len + 2 + extra / 2.0 + warmup + (steps - 1) / 2.0
    # drain
    while not eng.idle():
        eng.step()
    eng.take_finished()
    return dt, ctx


def prefill_run(eng, tokens, vocab, reps=3):
    import numpy as np
    import torch
    rng = np.random.default_rng(7)
    times = []
    for r in range(reps + 1):
        eng.add_request(rng.integers(3, vocab, size=tokens).tolist(), max_new_tokens=1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        info = eng.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        assert info.prefill_tokens == tokens
        eng.take_finished()
    return sorted(times[1:])[len(times[1:]) // 2]     # median, first one is warm-up


def measured_peaks():
    """What this GPU does in this run, beside the published peaks: GB/s of a copy kernel (1 GiB read and
    written), GB/s of a read-only kernel over 2 GiB, and TFLOP/s of a loop of bfloat16 matrix instructions
    that touches no memory.  Median of five launches each, timed by device events."""
    import torch
    from kvcm_amd import ops
    src = torch.zeros(1 << 29, dtype=torch.int32, device="cuda:0")       # 2 GiB
    dst = torch.empty(1 << 28, dtype=torch.int32, device="cuda:0")       # 1 GiB
    sink = torch.zeros(256, dtype=torch.float32, device="cuda:0")

    def timed(fn):
        ms = []
        for _ in range(6):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            b.synchronize()
            ms.append(a.elapsed_time(b))
        return sorted(ms[1:])[2] * 1e-3

    copy_s = timed(lambda: ops.probe_copy(src[:1 << 28], dst, grid=4096))
    read_s = timed(lambda: ops.probe_read(src, sink, grid=4096))
    flops = []
    mfma_s = timed(lambda: flops.append(ops.probe_mfma(20000, sink, grid=2048)))
    out = {"hbm_copy_GBs": round(2 * (1 << 30) / copy_s / 1e9, 1), "hbm_read_GBs": round((1 << 31) / read_s / 1e9, 1),
           "mfma_bf16_TFLOPs": round(flops[-1] / mfma_s / 1e12, 1)}
    del src, dst
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--sizes", default="tinyllama-1.1b", help="layer sizes by name (tinyllama-1.1b, llama-2-7b, llama-3-8b)")
    ap.add_argument("--tune-products", default="off", choices=["off", "heuristic", "all"],
                    help="which of the vendor library's algorithms the many-row products of prompt steps run: its first "
                         "choice (the engine's default, and this program's: the figures are a default engine's), the "
                         "fastest of its choices, or the fastest of all; timed at a shape's first use, before anything "
                         "is measured (tens of milliseconds per shape: worth it for shapes that run thousands of times)")
    ap.add_argument("--context-limit", type=int, default=0,
                    help="most tokens a request may hold; sizes the cache pool (default: 2,048, or what --prompt-len, "
                         "--warmup and --steps need if that is more)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--only-prefill", action="store_true",
                    help="run nothing but the 2,048-token prefill (for a profiler); prints its record alone")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="tokens of the prefill measurement (2,048 in the record; other lengths for sweeps)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus N with N > 1 is not supported")
        sys.exit(2)

    # a whole prompt fits a step beside the decoding requests
    budget = max(4096, args.prompt_len + args.batch, args.prefill_tokens + 64)
    needed = args.prompt_len + args.warmup + args.steps + 24 + prompt_step_count(args.batch, args.prompt_len, budget)
    limit = args.context_limit or max(2048, -(-needed // 64) * 64, -(-args.prefill_tokens // 64) * 64)
    if needed > limit:
        print("bench.py: --prompt-len %d plus the decoded tokens does not fit --context-limit %d" % (args.prompt_len, limit))
        sys.exit(2)

    import torch
    from kvcm_amd.config.model_config import LlamaConfig
    from kvcm_amd.weights.random_init import random_tensors

    from kvcm_amd.cli.common import NAMED_SIZES
    if args.sizes not in NAMED_SIZES:
        print("bench.py: unknown --sizes %r; known: %s" % (args.sizes, sorted(NAMED_SIZES)))
        sys.exit(2)
    sizes = dict(SIZES if args.sizes == "tinyllama-1.1b" else NAMED_SIZES[args.sizes])
    label = {"tinyllama-1.1b": "TinyLlama-1.1B", "llama-2-7b": "Llama-2-7B", "llama-3-8b": "Llama-3-8B"}.get(args.sizes, args.sizes)
    full_layers = sizes["num_hidden_layers"]
    if args.layers:
        sizes["num_hidden_layers"] = args.layers
    cfg = LlamaConfig.from_dict(sizes)
    dt = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    tensors = random_tensors("LlamaForCausalLM", cfg, seed=0, dtype=dt, device="cuda:0")
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers

    def roofline(batch, seconds_per_step, ctx):
        # the bytes are the loaded model's and its cache storages' own count (every weight the step uses once,
        # the embedding rows of its tokens, the keys and values of the live requests), not a formula of sizes
        achieved = eng.runner.step_bytes([ctx] * batch) / seconds_per_step / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_GBS, 4)}

    # the pool holds every request of the largest batch at the context limit
    seqs = args.batch if (args.no_points or args.only_prefill) else max(64, args.batch)
    eng = build_engine(cfg, args.dtype, max_num_seqs=seqs, max_batched_tokens=budget, tensors=tensors, context_limit=limit,
                       tune_products=args.tune_products)
    del tensors
    torch.cuda.empty_cache()

    def prefill_record():
        T = args.prefill_tokens
        sec = prefill_run(eng, T, V)
        flops = eng.model.step_flops(T, 1, T * (T + 1) // 2)      # the parts' own count: products, and q.k and p.v
        return {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                "frac": round(flops / sec / PEAK_FLOPS[key], 4)}

    def tuning_log():   # which shapes were tuned, the first choice's and the kept algorithm's microseconds
        if os.environ.get("KVCM_BENCH_TUNING_LOG"):
            from kvcm_amd import ops
            for row in ops.library_tuning_log:
                print("tuned M=%d N=%d K=%d: %.1f -> %.1f us (%d candidates)" % row, file=sys.stderr)

    if args.only_prefill:
        print(json.dumps({"prefill": prefill_record()}), flush=True)
        tuning_log()
        return

    seconds, ctx = decode_run(eng, args.batch, args.prompt_len, args.steps, args.warmup, V)
    value = args.batch * args.steps / seconds
    out = {
        "metric": "decode tok/s at batch %d (%s sizes, %d-token prompts)" % (args.batch, label, args.prompt_len),
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(1e3 * seconds / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": key, "data": "synthetic",
        "config": {"model": "%s sizes, random weights N(0,0.02)" % label, "global_batch": args.batch,
                   "seq_len": args.prompt_len, "parallelism": "single GPU", "layers": L, "layers_full": full_layers,
                   "hidden": H, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": I, "vocab": V, "kv_block": 16,
                   "context_limit": limit, "generated": args.warmup + args.steps,
                   "tune_products": args.tune_products},
        "roofline": roofline(args.batch, seconds / args.steps, ctx),
    }
    if not args.no_points:
        points = {}
        for b, k in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            s, c = decode_run(eng, b, args.prompt_len, k, min(args.warmup, 8), V, seed=10 + b)
            points[f"decode_b{b}"] = round(b * k / s, 1)
            points[f"decode_b{b}_ms"] = round(1e3 * s / k, 4)
            points[f"decode_b{b}_hbm_frac"] = roofline(b, s / k, c)["frac"]
        out["points"] = points
        out["prefill"] = prefill_record()
        # beside the published peaks the fractions above are taken against: what this GPU reached in this run
        out["measured"] = measured_peaks()
    print(json.dumps(out), flush=True)
    tuning_log()


if __name__ == "__main__":
    main()
