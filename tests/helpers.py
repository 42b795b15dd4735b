"""Shared by the GPU tests: the two tiny configurations, model folders with random weights whose
attention is sharp enough to show positional faults, and the schedules a trace is replayed in."""
import json
import os

import numpy as np
import torch

import plain_llama as plain

# Two tiny configurations that differ in every size and option.
TINY_A = dict(architectures=["LlamaForCausalLM"], vocab_size=256, hidden_size=64, intermediate_size=176,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY_B = dict(architectures=["LlamaForCausalLM"], vocab_size=384, hidden_size=96, intermediate_size=256,
              num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
              max_position_embeddings=256, rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=True)
# head_dim need not be hidden/heads, sizes need not be powers of two
TINY_C = dict(architectures=["LlamaForCausalLM"], vocab_size=331, hidden_size=80, intermediate_size=136,
              num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=3, head_dim=48,
              max_position_embeddings=512, rope_theta=250000.0, rms_norm_eps=3e-6, tie_word_embeddings=False)
# sizes that the matrix-core kernels of the bfloat16 path take (head_dim 64, K a multiple of 64 and
# long enough to be split): what the other three run through the general kernels, this one runs
# through the kernels a served model meets, with contexts beyond one chunk of 256 and one segment of 1,024 keys
TINY_D = dict(architectures=["LlamaForCausalLM"], vocab_size=300, hidden_size=256, intermediate_size=320,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
              max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
# the other head size of the matrix-core kernels (128), a group of three query heads per KV head,
# pages of 32, an odd vocabulary
TINY_E = dict(architectures=["LlamaForCausalLM"], vocab_size=1001, hidden_size=192, intermediate_size=272,
              num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=2, head_dim=128,
              max_position_embeddings=512, rope_theta=50000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
BLOCK_SIZE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 32}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}
WEIGHT_SEED = {"A": 0, "B": 2, "C": 5, "D": 7, "E": 9}
# factor on the q and k projections: chosen per width so that scores have a spread of a few units
# in every configuration (they grow with hidden_size * sqrt(head_dim); a spread of tens would make
# the 32-bit rounding of the scores themselves, amplified by exp, the largest error in the test)
SHARPEN = {"A": 12.0, "B": 12.0, "C": 12.0, "D": 6.0, "E": 6.0}


def make_model_dir(path, raw, seed, dtype, sharpen=12.0):
    """Random N(0, 0.02) weights (norm weights 1 + 0.1 N so that the multiply matters), with the q
    and k projections scaled up so that attention scores spread over several units: a wrong
    position, a missing key or a stale page then changes the logits visibly."""
    from kvcm_amd.config.model_config import LlamaConfig
    from kvcm_amd.weights.random_init import random_tensors
    from kvcm_amd.weights.safetensors_io import write_safetensors
    cfg = LlamaConfig.from_dict(raw)
    tensors = random_tensors("LlamaForCausalLM", cfg, seed, torch.float32, std=0.02, norm_jitter=0.1)
    for name in tensors:
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            tensors[name] = tensors[name] * sharpen
        if "embed_tokens" in name:
            tensors[name] = tensors[name] * 20.0        # residual stream of order one
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors)
    return path


def requests_for(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, raw["vocab_size"], size=n).tolist() for i, n in enumerate(lengths)}


# ------------------------------------------------------------------------------ schedules
def schedule_whole(reqs):
    """Each request alone, whole, every position wanted."""
    return [{"step": k, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for k, (rid, toks) in enumerate(reqs.items())]


def schedule_tail_singly(reqs, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps, k = [], 0
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": k, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        k += 1
        for i in range(head, len(toks)):
            steps.append({"step": k, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
            k += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def schedule_portions(reqs, sizes=(7, 2, 16, 3, 5, 2, 33, 4, 2, 11)):
    """Portions of changing size, down to two tokens."""
    steps, k, c = [], 0, 0
    for rid, toks in reqs.items():
        pos = 0
        while pos < len(toks):
            n = min(sizes[c % len(sizes)], len(toks) - pos)
            c += 1
            last = pos + n == len(toks)
            steps.append({"step": k, "entries": [{"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            pos += n
            k += 1
    return steps


def schedule_mixed(reqs, seed=0, max_live=4, sizes=(9, 2, 5, 17, 3, 2, 6)):
    """Up to ``max_live`` live requests: in every step portions of some beside single tokens of
    others; a request may sit a step out; finished requests hand their pages to new ones."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs.items())
    live = {}                       # rid -> position reached
    steps, k, c = [], 0, 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.25:
                continue             # left out of this step, goes on later
            toks = reqs[rid]
            pos = live[rid]
            decode_phase = pos >= max(1, len(toks) - 12)
            n = 1 if decode_phase else min(sizes[c % len(sizes)], len(toks) - pos)
            c += 1
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))})
            live[rid] = pos + n
            if live[rid] == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": k, "entries": entries, "end": ended})
            k += 1
    return steps


def tokens_needed(reqs, max_live=4):
    """Pool size for a trace: the ``max_live`` longest requests, each rounded up to 64."""
    sizes = sorted((-(-len(t) // 64) * 64 for t in reqs.values()), reverse=True)
    return sum(sizes[:max_live])


def replay(replayer, steps, reqs):
    """-> {request id: logits [len, V]} gathered from the wanted rows of every step."""
    V = replayer.vocab_size
    out = {rid: np.full((len(t), V), np.nan, dtype=np.float32) for rid, t in reqs.items()}
    pos = {rid: 0 for rid in reqs}
    for rec in steps:
        logits = replayer.step(rec)
        row = 0
        for e in rec["entries"]:
            for w in e["want"]:
                out[e["id"]][pos[e["id"]] + w] = logits[row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
        assert (logits is None and row == 0) or row == logits.shape[0]
    return out


def plain_logits(model_dir, reqs, bf16):
    pm = plain.load_model_dir(model_dir, plain.round_bf16 if bf16 else None)
    return {rid: pm.logits(t) for rid, t in reqs.items()}, pm


def first_difference(got, ref, tol):
    """(request, position, error) of the first position whose logits differ by more than tol."""
    for rid in ref:
        err = np.abs(got[rid].astype(np.float64) - ref[rid]).max(axis=1)
        bad = np.nonzero(~(err <= tol))[0]
        if len(bad):
            return rid, int(bad[0]), float(err[bad[0]])
    return None


# ------------------------------------------------------------- inputs where the order of rounding shows
def norm_rounding_cases(rows=4, width=256, seed=3):
    """(x float32 rows, w on the bfloat16 grid) for an RMS norm: plenty of elements for which
    round(w * round(x * inv)) differs from a single rounding after the multiply, and none where x * inv
    lies so close to a rounding boundary of bfloat16 that 32-bit arithmetic could decide it the other
    way than exact arithmetic (those elements are nudged away)."""
    rng = np.random.default_rng(seed)
    x = rng.normal(size=(rows, width)).astype(np.float32).astype(np.float64)
    w = plain.round_bf16(1.0 + 0.3 * rng.normal(size=width))
    for _ in range(4):
        inv = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
        y = x * inv
        lo = plain.round_bf16(y)
        ulp = np.abs(lo) * 2.0 ** -8 + 1e-30
        frac = np.abs(y - lo) / ulp                              # 0 .. 0.5 of a step away from the rounded value
        near = frac > 0.49                                       # too close to the midpoint between two grid values
        x = np.where(near, x * (1.0 + 2.0 ** -9), x).astype(np.float32).astype(np.float64)
        p = w * lo
        pl = plain.round_bf16(p)
        near2 = np.abs(p - pl) / (np.abs(pl) * 2.0 ** -8 + 1e-30) > 0.49
        x = np.where(near2, x * (1.0 - 2.0 ** -9), x).astype(np.float32).astype(np.float64)
    return x, w


def swiglu_rounding_cases(rows=3, width=200, seed=4):
    """(gate, up) on the bfloat16 grid with silu(gate) safely away from rounding boundaries."""
    rng = np.random.default_rng(seed)
    g = plain.round_bf16(rng.normal(size=(rows, width)) * 2.0)
    u = plain.round_bf16(rng.normal(size=(rows, width)) * 2.0)
    for _ in range(4):
        s = g / (1.0 + np.exp(-g))
        sl = plain.round_bf16(s)
        near = np.abs(s - sl) / (np.abs(sl) * 2.0 ** -8 + 1e-30) > 0.47
        g = np.where(near, plain.round_bf16(g * (1.0 + 2.0 ** -6)), g)
        p = sl * u
        pl = plain.round_bf16(p)
        near2 = np.abs(p - pl) / (np.abs(pl) * 2.0 ** -8 + 1e-30) > 0.49
        u = np.where(near2, plain.round_bf16(u * (1.0 + 2.0 ** -6)), u)
    return g, u
