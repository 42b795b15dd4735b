"""Parts and architectures that the package does not have, defined here and registered from
outside: a mixer with per-request state of its own, and a model whose layer list runs a layer
twice and lets a layer read another layer's cache.  Nothing in the package changes for them."""
import json
import os
from dataclasses import asdict, dataclass

import numpy as np
import pytest
import torch

import plain_llama as plain

pytestmark = pytest.mark.gpu


# --------------------------------------------------------------- a mixer with its own state
def _register_toy():
    from kvcm_amd.parts.base import LayerSpec, Mixer, ModelSpec, ParamSpec, PartSpec, StateNeed
    from kvcm_amd.registry import ARCHITECTURES, MIXERS, Architecture

    if "toy_decay_state" in MIXERS:
        return

    @MIXERS.register("toy_decay_state")
    class DecayState(Mixer):
        """s_t = decay * s_{t-1} + W_in h_t ; out_t = W_out s_t.  The state of a request lives in
        its slot between steps; rows of one request are taken in order."""

        def param_specs(self):
            H, D = self.ctx.hidden_size, self.params["state_size"]
            return [ParamSpec("w_in", ((self.prefix + "in_proj.weight", (D, H)),)),
                    ParamSpec("w_out", ((self.prefix + "out_proj.weight", (H, D)),))]

        def cache_need(self):
            return StateNeed((self.params["state_size"],), torch.float32)

        def forward(self, step, h):
            slots = self.cache.slots(self.cache_index)
            out = step.ws("mixer_out", (step.rows, self.ctx.hidden_size))
            u = h.float() @ self.w["w_in"].float().T
            for s in range(step.real_seqs):
                lo, hi = int(step.host_run_start[s]), int(step.host_run_start[s + 1])
                slot = int(step.host_state_slots[s])
                state = torch.zeros_like(slots[slot]) if int(step.host_seq_start[s]) == 0 else slots[slot].clone()
                for r in range(lo, hi):
                    state = self.params["decay"] * state + u[r]
                    out[r] = (self.w["w_out"].float() @ state).to(out.dtype)
                slots[slot] = state
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        width: int
        inner: int
        depth: int
        state_size: int
        decay: float
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("vocab_size", "width", "inner", "depth", "state_size", "decay", "eps")})

        def to_dict(self):
            return asdict(self)

    def spec(cfg):
        layers = tuple(LayerSpec(
            name=f"b{l}", block="prenorm_residual",
            parts={"norm_mixer": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, f"blocks.{l}.n1."),
                   "mixer": PartSpec("toy_decay_state", {"state_size": cfg.state_size, "decay": cfg.decay}, f"blocks.{l}.mix."),
                   "norm_ffn": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, f"blocks.{l}.n2."),
                   "ffn": PartSpec("swiglu", {"intermediate_size": cfg.inner}, f"blocks.{l}.mlp.")})
            for l in range(cfg.depth))
        return ModelSpec("ToyStateForCausalLM", cfg.width, cfg.vocab_size,
                         PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "emb."), layers,
                         tuple(range(cfg.depth)), PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, "out_norm."),
                         PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": True}, "head."))

    ARCHITECTURES.register("ToyStateForCausalLM", Architecture("ToyStateForCausalLM", ToyConfig, spec))


def _toy_plain_logits(raw, t, tokens):
    x = plain.embedding(t["emb.weight"], tokens)
    for l in range(raw["depth"]):
        p = f"blocks.{l}."
        h = plain.rms_norm(x, t[p + "n1.weight"], raw["eps"])
        u = h @ t[p + "mix.in_proj.weight"].T
        state = np.zeros(raw["state_size"])
        a = np.zeros_like(x)
        for r in range(len(tokens)):
            state = raw["decay"] * state + u[r]
            a[r] = t[p + "mix.out_proj.weight"] @ state
        x = x + a
        h = plain.rms_norm(x, t[p + "n2.weight"], raw["eps"])
        gu = np.concatenate([plain.linear(h, t[p + "mlp.gate_proj.weight"]), plain.linear(h, t[p + "mlp.up_proj.weight"])], -1)
        x = x + plain.linear(plain.swiglu(gu), t[p + "mlp.down_proj.weight"])
    return plain.rms_norm(x, t["out_norm.weight"], raw["eps"]) @ t["emb.weight"].T


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    _register_toy()
    from kvcm_amd import Engine, EngineConfig
    from kvcm_amd.engine.replay import TraceReplayer
    from kvcm_amd.registry import ARCHITECTURES
    from kvcm_amd.weights.random_init import write_model_dir

    raw = dict(architectures=["ToyStateForCausalLM"], vocab_size=97, width=40, inner=56, depth=2, state_size=24,
               decay=0.9, eps=1e-5)
    cfg = ARCHITECTURES.get("ToyStateForCausalLM").config_class.from_dict(raw)
    d = write_model_dir(str(tmp_path / "toy"), "ToyStateForCausalLM", cfg, seed=4, dtype=torch.float32, std=0.3, norm_jitter=0.1)
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    rng = np.random.default_rng(0)
    reqs = {"x": rng.integers(0, 97, size=23).tolist(), "y": rng.integers(0, 97, size=9).tolist(),
            "z": rng.integers(0, 97, size=14).tolist()}
    ref = {k: _toy_plain_logits(raw, t, v) for k, v in reqs.items()}

    rp = TraceReplayer(d, "float32", max_tokens=256)
    assert [g.kind for g in rp.core.groups] == ["state"]          # no pages at all, one slot per request
    # whole, then in portions beside other requests: the state carries over between steps
    whole = rp.step({"step": 0, "entries": [{"id": "x", "tokens": reqs["x"], "want": list(range(23))}], "end": ["x"]})
    np.testing.assert_allclose(whole, ref["x"], atol=2e-4)
    got = {k: [] for k in reqs}
    steps = [[("x", 0, 5), ("y", 0, 9)], [("x", 5, 7), ("z", 0, 2)], [("z", 2, 14)], [("x", 7, 8), ("z", 14, 14)],
             [("x", 8, 23)]]
    for k, entries in enumerate(steps):
        entries = [e for e in entries if e[2] > e[1]]
        ended = [rid for rid, lo, hi in entries if hi == len(reqs[rid])]
        out = rp.step({"step": k + 1, "entries": [{"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}
                                                  for rid, lo, hi in entries], "end": ended})
        row = 0
        for rid, lo, hi in entries:
            got[rid].append(out[row:row + hi - lo])
            row += hi - lo
    for rid in reqs:
        np.testing.assert_allclose(np.concatenate(got[rid]), ref[rid], atol=2e-4)
    assert rp.core.state_slots_free() == 8

    # and through the scheduler: greedy generation equals the plain toy
    eng = Engine(d, EngineConfig(dtype="float32", num_blocks=8, max_seq_len=64, max_num_seqs=4, max_batched_tokens=64,
                                 prefill_chunk=6, use_graphs=False))
    prompts = [reqs["y"], reqs["z"][:5]]
    outs = eng.generate(prompts, 6)
    for p, g in zip(prompts, outs):
        toks = list(p)
        for k in range(6):
            row = _toy_plain_logits(raw, t, toks)[-1]
            srt = np.sort(row)
            assert g[k] == int(np.argmax(row)) or srt[-1] - srt[-2] < 1e-4
            toks.append(g[k])


# ------------------------------------- a layer run twice, a layer reading another's cache
def test_layer_list_may_repeat_a_layer_and_share_a_cache(tmp_path):
    from kvcm_amd.engine.replay import TraceReplayer
    from kvcm_amd.parts.base import LayerSpec, ModelSpec, PartSpec
    from kvcm_amd.registry import ARCHITECTURES, Architecture
    from kvcm_amd.weights.random_init import write_model_dir

    @dataclass(frozen=True)
    class Cfg:
        vocab_size: int
        width: int
        heads: int
        kv_heads: int
        head_dim: int
        inner: int
        theta: float
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("vocab_size", "width", "heads", "kv_heads", "head_dim", "inner", "theta", "eps")})

        def to_dict(self):
            return asdict(self)

    def layer(cfg, name, prefix, cache_from=None):
        attn = {"num_heads": cfg.heads, "num_kv_heads": cfg.kv_heads, "head_dim": cfg.head_dim, "scale": cfg.head_dim ** -0.5,
                "window": 0, "position": PartSpec("rotary", {"theta": cfg.theta, "dim": cfg.head_dim})}
        return LayerSpec(name, "prenorm_residual",
                         {"norm_mixer": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix + "n1."),
                          "mixer": PartSpec("gqa_attention", attn, prefix + "attn."),
                          "norm_ffn": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix + "n2."),
                          "ffn": PartSpec("swiglu", {"intermediate_size": cfg.inner}, prefix + "mlp.")}, cache_from)

    def spec(cfg):
        layers = (layer(cfg, "first", "l0."), layer(cfg, "reader", "l1.", cache_from="first"))
        return ModelSpec("SharedCacheForCausalLM", cfg.width, cfg.vocab_size,
                         PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "emb."), layers,
                         (0, 1, 1),                                # the reader runs twice
                         PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, "norm."),
                         PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": False}, "head."))

    ARCHITECTURES.register("SharedCacheForCausalLM", Architecture("SharedCacheForCausalLM", Cfg, spec))
    raw = dict(architectures=["SharedCacheForCausalLM"], vocab_size=120, width=48, heads=4, kv_heads=2, head_dim=16,
               inner=80, theta=5000.0, eps=1e-5)
    cfg = Cfg.from_dict(raw)
    d = write_model_dir(str(tmp_path / "shared"), "SharedCacheForCausalLM", cfg, seed=9, dtype=torch.float32, std=0.15,
                        norm_jitter=0.1)
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    toks = np.random.default_rng(1).integers(0, 120, size=37).tolist()

    n, pos = len(toks), np.arange(len(toks))
    x = plain.embedding(t["emb.weight"], toks)
    kv = None
    for pre in ("l0.", "l1.", "l1."):
        h = plain.rms_norm(x, t[pre + "n1.weight"], 1e-5)
        q = plain.rotary(plain.linear(h, t[pre + "attn.q_proj.weight"]).reshape(n, 4, 16), pos, 5000.0)
        if pre == "l0.":
            kv = (plain.rotary(plain.linear(h, t[pre + "attn.k_proj.weight"]).reshape(n, 2, 16), pos, 5000.0),
                  plain.linear(h, t[pre + "attn.v_proj.weight"]).reshape(n, 2, 16))
        a = plain.attention(q, kv[0], kv[1], pos, pos, 0.25)
        x = x + plain.linear(a.reshape(n, 64), t[pre + "attn.o_proj.weight"])
        h = plain.rms_norm(x, t[pre + "n2.weight"], 1e-5)
        gu = np.concatenate([plain.linear(h, t[pre + "mlp.gate_proj.weight"]), plain.linear(h, t[pre + "mlp.up_proj.weight"])], -1)
        x = x + plain.linear(plain.swiglu(gu), t[pre + "mlp.down_proj.weight"])
    ref = plain.rms_norm(x, t["norm.weight"], 1e-5) @ t["head.weight"].T

    rp = TraceReplayer(d, "float32", max_tokens=64)
    assert len(rp.model.groups) == 1 and rp.model.groups[0].layers == ["first"]       # one cache, one owner
    assert rp.runner.storages[0].num_layers == 1
    a = rp.step({"step": 0, "entries": [{"id": "s", "tokens": toks[:20], "want": list(range(20))}], "end": []})
    b = rp.step({"step": 1, "entries": [{"id": "s", "tokens": toks[20:22], "want": [0, 1]}], "end": []})
    c = rp.step({"step": 2, "entries": [{"id": "s", "tokens": toks[22:], "want": list(range(15))}], "end": ["s"]})
    np.testing.assert_allclose(np.concatenate([a, b, c]), ref, atol=1e-4)
