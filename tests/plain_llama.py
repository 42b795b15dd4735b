"""A plain, slow Llama decoder in NumPy float64: whole sequences, no cache, no batching.

One function per part, each written from the formula the reference engine computes
(file:line given per function, relative to the reference checkout).  It shares no code
with the product package: tests compare the engine against it.

Two precision modes:
  * ``r16=None``        nothing is rounded (the oracle for the engine's 32-bit path);
  * ``r16=round_bf16``  values are rounded to bfloat16 exactly where the serving path
                        stores a 16-bit value (the reference stores fp16 at those points).
"""
import json
import math
import os
import struct

import numpy as np


# ----------------------------------------------------------------------------- rounding
def round_bf16(a):
    """Round-to-nearest-even to bfloat16, returned as float64."""
    f = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    u = f.view(np.uint32)
    # add half a step of the 16 bits that go (0x7FFF, and the kept part's last bit to break ties to even),
    # then drop them; 32-bit unsigned arithmetic, which wraps only for NaN patterns
    kept = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) & np.uint32(0xFFFF0000)
    return kept.view(np.float32).astype(np.float64).reshape(f.shape)


def _ident(a):
    return np.asarray(a, dtype=np.float64)


# ----------------------------------------------------------------------------- parts
def embedding(table, ids):
    """x[t,:] = float(table[ids[t],:]); no scaling, nothing added.  src/cuda/kernels.cu:27-32"""
    return np.asarray(table, dtype=np.float64)[np.asarray(ids, dtype=np.int64)]


def rms_norm(x, w, eps, r16=None):
    """ss = sum x^2; inv = 1/sqrt(ss/H + eps); out = w * round16(x*inv).

    eps is inside the root, the mean runs over the whole row, no mean is subtracted and the
    weight is a plain multiplier; the 16-bit cast happens before the weight multiply and the
    product is again a 16-bit value.  src/cuda/kernels.cu:34-49
    """
    r = r16 or _ident
    x = np.asarray(x, dtype=np.float64)
    inv = 1.0 / np.sqrt((x * x).sum(-1, keepdims=True) / x.shape[-1] + eps)
    return r(np.asarray(w, dtype=np.float64) * r(x * inv))


def linear(x, w, r16=None):
    """y = x @ w.T with w stored [out_features, in_features]; no bias; the accumulator is
    wide and the stored result 16-bit.  src/model/llama.cpp:45-52"""
    r = r16 or _ident
    return r(np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T)


def rotary_angles(positions, head_dim, theta):
    """inv_freq_j = 1/theta^(2j/hd) and angle = pos*inv_freq_j, both in float32.
    src/cuda/kernels.cu:60-63"""
    j = np.arange(head_dim // 2, dtype=np.float32)
    inv_freq = (np.float32(1.0) / np.power(np.float32(theta), (np.float32(2.0) * j) / np.float32(head_dim))).astype(np.float32)
    pos = np.asarray(positions, dtype=np.float32)[:, None]
    return (pos * inv_freq[None, :]).astype(np.float32).astype(np.float64)


def rotary(v, positions, theta, r16=None):
    """Rotate-half pairing (j, j+hd/2) over the full head_dim of every head.

    v: [T, heads, hd].  (a,b) = (v[j], v[j+hd/2]) -> (a cos - b sin, b cos + a sin).
    src/cuda/kernels.cu:51-70
    """
    r = r16 or _ident
    v = np.asarray(v, dtype=np.float64)
    hd = v.shape[-1]
    ang = rotary_angles(positions, hd, theta)[:, None, :]
    cs, sn = np.cos(ang), np.sin(ang)
    a, b = v[..., : hd // 2], v[..., hd // 2:]
    return r(np.concatenate([a * cs - b * sn, b * cs + a * sn], axis=-1))


def attention(q, k, v, positions_q, positions_k, scale, window=0, r16=None):
    """Causal attention of query rows over keys, one KV head per group of query heads.

    q: [Tq, nh, hd], k/v: [Tk, nkv, hd].  Row r sees keys with position <= its own
    (context_len = pos+1 is the only mask); query head h reads KV head h // (nh/nkv); the
    scale multiplies q before the dot product; softmax in wide precision; the output is one
    16-bit store.  src/cuda/paged_attention.cu:94-100 (q*scale), 107-128 (scores),
    131-147 (softmax), 150-183 (PV, divide by the sum).
    ``window`` (> 0) additionally hides keys with pos_q - pos_k >= window; the reference has no
    window, the engine's cache groups do.
    """
    r = r16 or _ident
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    nh, nkv = q.shape[1], k.shape[1]
    group = nh // nkv
    pq = np.asarray(positions_q)[:, None]
    pk = np.asarray(positions_k)[None, :]
    visible = pk <= pq
    if window and window > 0:
        visible &= (pq - pk) < window
    out = np.zeros_like(q)
    for h in range(nh):
        s = (q[:, h, :] * scale) @ k[:, h // group, :].T
        s = np.where(visible, s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        out[:, h, :] = (p @ v[:, h // group, :]) / p.sum(-1, keepdims=True)
    return r(out)


def swiglu(gate_up, r16=None):
    """act = round16( round16(silu(g)) * u ), silu(g) = g / (1 + exp(-g)); the row holds the
    gate half first and the up half second.  src/cuda/kernels.cu:72-82"""
    r = r16 or _ident
    gu = np.asarray(gate_up, dtype=np.float64)
    inter = gu.shape[-1] // 2
    g, u = gu[..., :inter], gu[..., inter:]
    return r(r(g / (1.0 + np.exp(-g))) * u)


def argmax_rows(logits):
    """Lowest index among equal maxima.  src/cuda/kernels.cu:90-119"""
    return np.argmax(np.asarray(logits), axis=-1).astype(np.int64)


# ----------------------------------------------------------------------------- sampling
_M64 = (1 << 64) - 1


def _mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def gumbel_uniforms(seed, request_id, token_index, vocab):
    """u_j in (0,1), a pure function of (seed, request, index of the generated token, j).
    The reference samples greedily only; this counter-based draw is the engine's own."""
    h = _mix64((seed + 0x9E3779B97F4A7C15 * (request_id + 1)) & _M64)
    h = _mix64(h ^ ((token_index * 0xBF58476D1CE4E5B9) & _M64))
    out = np.empty(vocab, dtype=np.float64)
    for j in range(vocab):
        out[j] = ((_mix64((h + j) & _M64) >> 41) + 0.5) / float(1 << 23)
    return out


def sample_row(logits, temperature, seed, request_id, token_index):
    """temperature 0 -> argmax; otherwise argmax_j(logit_j / T - log(-log u_j))."""
    logits = np.asarray(logits, dtype=np.float64)
    if temperature <= 0:
        return int(np.argmax(logits)), None
    u = gumbel_uniforms(seed, request_id, token_index, logits.shape[0])
    score = logits / temperature - np.log(-np.log(u))
    order = np.argsort(-score, kind="stable")
    return int(order[0]), float(score[order[0]] - score[order[1]])


# ----------------------------------------------------------------- seeded random weights
def counter_normal(seed, name, count):
    """Standard normal values of the random-weights rule for one tensor, as float32: a counter-based
    generator keyed by (seed, tensor name, element index), written here from the rule's description
    (SplitMix64 mixing, FNV-1a of the name, Box-Muller in double precision) and sharing no code with
    the engine's.  The reference has no random weights (src/main_bench.cpp:6-7)."""
    mask = (1 << 64) - 1

    def mix_int(z):
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)

    def mix(z):
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))

    h = 0xCBF29CE484222325
    for byte in name.encode():
        h = ((h ^ byte) * 0x100000001B3) & mask
    key = mix_int(mix_int(seed & mask) ^ h)
    with np.errstate(over="ignore"):
        z1 = mix(np.uint64(key) + np.arange(1, count + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
        z2 = mix(z1)
    u1 = ((z1 >> np.uint64(12)).astype(np.float64) + 0.5) / 2.0 ** 52
    u2 = (z2 >> np.uint64(12)).astype(np.float64) / 2.0 ** 52
    return (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def counter_weight(seed, name, shape, std=0.02, vector=False, norm_jitter=0.0):
    """A tensor of the rule: float32(std * n) for matrices and tables, float32(1 + norm_jitter * n) for
    norm weights, in float32 arithmetic."""
    n = counter_normal(seed, name, int(np.prod(shape)))
    if vector:
        return (np.float32(1.0) + np.float32(norm_jitter) * n).reshape(shape) if norm_jitter else np.ones(shape, np.float32)
    return (np.float32(std) * n).reshape(shape)


# ----------------------------------------------------------------------------- the model
class PlainLlama:
    """Holds float64 copies of a checkpoint's tensors under their checkpoint names."""

    def __init__(self, cfg, tensors, r16=None):
        self.cfg = dict(cfg)
        self.t = {k: np.asarray(v, dtype=np.float64) for k, v in tensors.items()}
        self.r16 = r16
        c = self.cfg
        self.H = c["hidden_size"]
        self.nh = c["num_attention_heads"]
        self.nkv = c.get("num_key_value_heads", self.nh)
        self.hd = c.get("head_dim") or self.H // self.nh
        self.L = c["num_hidden_layers"]
        self.theta = float(c.get("rope_theta", 10000.0))
        self.eps = float(c.get("rms_norm_eps", 1e-5))
        self.tied = bool(c.get("tie_word_embeddings", False))

    def layer(self, l, x, positions):
        """One pre-norm residual block.  src/model/llama.cpp:104-124"""
        t, r = self.t, self.r16
        p = f"model.layers.{l}."
        T = x.shape[0]
        h = rms_norm(x, t[p + "input_layernorm.weight"], self.eps, r)
        q = linear(h, t[p + "self_attn.q_proj.weight"], r).reshape(T, self.nh, self.hd)
        k = linear(h, t[p + "self_attn.k_proj.weight"], r).reshape(T, self.nkv, self.hd)
        v = linear(h, t[p + "self_attn.v_proj.weight"], r).reshape(T, self.nkv, self.hd)
        q = rotary(q, positions, self.theta, r)
        k = rotary(k, positions, self.theta, r)
        a = attention(q, k, v, positions, positions, 1.0 / math.sqrt(self.hd), 0, r)
        x = x + linear(a.reshape(T, self.nh * self.hd), t[p + "self_attn.o_proj.weight"], r)
        h = rms_norm(x, t[p + "post_attention_layernorm.weight"], self.eps, r)
        gu = np.concatenate([linear(h, t[p + "mlp.gate_proj.weight"], r),
                             linear(h, t[p + "mlp.up_proj.weight"], r)], axis=-1)
        x = x + linear(swiglu(gu, r), t[p + "mlp.down_proj.weight"], r)
        return x

    def logits(self, tokens, rows=None):
        """Logits [T, V] at every position of one whole sequence (``rows``: at these positions only;
        the final norm and the head work row by row).  src/model/llama.cpp:84-128"""
        t, r = self.t, self.r16
        positions = np.arange(len(tokens))
        x = embedding(t["model.embed_tokens.weight"], tokens)
        for l in range(self.L):
            x = self.layer(l, x, positions)
        if rows is not None:
            x = x[np.asarray(rows, dtype=np.int64)]
        h = rms_norm(x, t["model.norm.weight"], self.eps, r)
        head = t["model.embed_tokens.weight"] if self.tied else t["lm_head.weight"]
        return np.asarray(h, dtype=np.float64) @ head.T  # logits stay wide

    def logits_of_many(self, sequences, rows):
        """``logits(sequences[i], rows[i])`` for many whole sequences at once, for tests with hundreds of
        requests at real widths: everything that works row by row (norms, projections, rotation by each
        row's own position, SwiGLU, head) runs on the sequences' rows stacked, attention runs per sequence
        as in ``layer``.  Still no cache and no batching of attention; the same part functions."""
        t, r = self.t, self.r16
        lens = [len(s) for s in sequences]
        starts = np.concatenate([[0], np.cumsum(lens)])
        positions = np.concatenate([np.arange(n) for n in lens])
        x = embedding(t["model.embed_tokens.weight"], np.concatenate([np.asarray(s, dtype=np.int64) for s in sequences]))
        T = x.shape[0]
        for l in range(self.L):
            p = f"model.layers.{l}."
            h = rms_norm(x, t[p + "input_layernorm.weight"], self.eps, r)
            q = rotary(linear(h, t[p + "self_attn.q_proj.weight"], r).reshape(T, self.nh, self.hd), positions, self.theta, r)
            k = rotary(linear(h, t[p + "self_attn.k_proj.weight"], r).reshape(T, self.nkv, self.hd), positions, self.theta, r)
            v = linear(h, t[p + "self_attn.v_proj.weight"], r).reshape(T, self.nkv, self.hd)
            a = np.concatenate([attention(q[lo:hi], k[lo:hi], v[lo:hi], positions[lo:hi], positions[lo:hi],
                                          1.0 / math.sqrt(self.hd), 0, r) for lo, hi in zip(starts[:-1], starts[1:])])
            x = x + linear(a.reshape(T, self.nh * self.hd), t[p + "self_attn.o_proj.weight"], r)
            h = rms_norm(x, t[p + "post_attention_layernorm.weight"], self.eps, r)
            gu = np.concatenate([linear(h, t[p + "mlp.gate_proj.weight"], r), linear(h, t[p + "mlp.up_proj.weight"], r)], axis=-1)
            x = x + linear(swiglu(gu, r), t[p + "mlp.down_proj.weight"], r)
        head = t["model.embed_tokens.weight"] if self.tied else t["lm_head.weight"]
        out = []
        for lo, want in zip(starts[:-1], rows):
            h = rms_norm(x[lo + np.asarray(want, dtype=np.int64)], t["model.norm.weight"], self.eps, r)
            out.append(np.asarray(h, dtype=np.float64) @ head.T)
        return out

    def generate(self, prompt, max_new_tokens, temperature=0.0, seed=0, request_id=0):
        toks = list(prompt)
        margins = []
        for i in range(max_new_tokens):
            row = self.logits(toks)[-1]
            nxt, margin = sample_row(row, temperature, seed, request_id, i)
            if margin is None:
                srt = np.sort(row)
                margin = float(srt[-1] - srt[-2])
            margins.append(margin)
            toks.append(nxt)
        return toks[len(prompt):], margins


# ----------------------------------------------------------------------------- file reading
_ST_DTYPES = {"F32": np.float32, "F16": np.float16, "F64": np.float64, "I32": np.int32, "I64": np.int64}


def read_safetensors(path):
    """Minimal reader of the container: u64 header length, JSON header, raw little-endian data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        base = 8 + n
        out = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            lo, hi = info["data_offsets"]
            f.seek(base + lo)
            raw = f.read(hi - lo)
            if info["dtype"] == "BF16":
                u = np.frombuffer(raw, dtype=np.uint16).astype(np.uint32) << 16
                arr = u.view(np.float32)
            else:
                arr = np.frombuffer(raw, dtype=_ST_DTYPES[info["dtype"]])
            out[name] = arr.reshape(info["shape"]).astype(np.float64)
    return out


def load_model_dir(path, r16=None):
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    return PlainLlama(cfg, read_safetensors(os.path.join(path, "model.safetensors")), r16)
