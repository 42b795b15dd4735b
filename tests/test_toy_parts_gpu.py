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

    # and through the scheduler, with the engine's default options for recorded steps (graphs, launch
    # lists): this mixer reads the step's host arrays, says nothing about being capturable, and so
    # every step of the model runs directly; greedy generation equals the plain toy
    eng = Engine(d, EngineConfig(dtype="float32", num_blocks=8, max_seq_len=64, max_num_seqs=4, max_batched_tokens=64,
                                 prefill_chunk=6))
    assert eng.config.use_graphs and eng.config.use_programs
    assert eng.decode_graphs is None and eng.programs is None and eng.model.not_capturable() == ["DecayState"]
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
    assert len(rp.model.groups) == 1 and rp.model.groups[0].layers == [("first", "mixer")]       # one cache, one owner
    assert rp.runner.storages[0].num_layers == 1
    a = rp.step({"step": 0, "entries": [{"id": "s", "tokens": toks[:20], "want": list(range(20))}], "end": []})
    b = rp.step({"step": 1, "entries": [{"id": "s", "tokens": toks[20:22], "want": [0, 1]}], "end": []})
    c = rp.step({"step": 2, "entries": [{"id": "s", "tokens": toks[22:], "want": list(range(15))}], "end": ["s"]})
    np.testing.assert_allclose(np.concatenate([a, b, c]), ref, atol=1e-4)


# ------ full and windowed attention layers side by side, a routed feed-forward, another position encoding
def _register_mixed():
    from kvcm_amd.parts.base import FeedForward, LayerSpec, ModelSpec, ParamSpec, PartSpec, PositionEncoding
    from kvcm_amd.registry import ARCHITECTURES, FEED_FORWARDS, POSITIONS, Architecture

    if "toy_top1_experts" in FEED_FORWARDS:
        return

    @POSITIONS.register("toy_damped")
    class Damped(PositionEncoding):
        """q[.., d] and k[.., d] are multiplied by cos(position * base^(-d / head_dim)): absolute, not a
        rotation, so the engine may not fuse it; v and the page write are left to the caller."""

        def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
            d = torch.arange(head_dim, dtype=torch.float32, device=qkv.device)
            freq = torch.pow(torch.tensor(float(self.params["base"]), device=qkv.device), -d / head_dim)
            factor = torch.cos(step.positions[:step.rows].float()[:, None] * freq[None, :])          # [rows, hd]
            heads = num_heads + num_kv_heads
            view = qkv[:step.rows, :heads * head_dim].view(step.rows, heads, head_dim)
            view.copy_((view.float() * factor[:, None, :]).to(qkv.dtype))
            return False

    @FEED_FORWARDS.register("toy_top1_experts")
    class Top1Experts(FeedForward):
        """The expert with the largest router logit (32-bit) alone runs: w2[e] relu(w1[e] h)."""

        def param_specs(self):
            H, E, I, pre = self.ctx.hidden_size, self.params["experts"], self.params["inner"], self.prefix
            return [ParamSpec("router", ((pre + "router.weight", (E, H)),)),
                    ParamSpec("w1", ((pre + "experts.w1", (E * I, H)),)),
                    ParamSpec("w2", ((pre + "experts.w2", (E * H, I)),))]

        def forward(self, step, h):
            H, E, I = self.ctx.hidden_size, self.params["experts"], self.params["inner"]
            out = step.ws("ffn_out", (step.rows, H))
            x = h[:step.rows].float()
            choice = (x @ self.w["router"].float().T).argmax(-1)
            w1, w2 = self.w["w1"].float().view(E, I, H), self.w["w2"].float().view(E, H, I)
            mid = torch.relu(torch.einsum("rih,rh->ri", w1[choice], x))
            out[:step.rows] = torch.einsum("rhi,ri->rh", w2[choice], mid).to(out.dtype)
            return out

    @dataclass(frozen=True)
    class MixedConfig:
        vocab_size: int
        width: int
        eps: float
        layers: tuple          # per layer: dict(heads, kv_heads, head_dim, window, position, ffn)

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["vocab_size"], raw["width"], raw["eps"], tuple(raw["layers"]))

        def to_dict(self):
            return {"vocab_size": self.vocab_size, "width": self.width, "eps": self.eps, "layers": list(self.layers)}

    def spec(cfg):
        layers = []
        for l, d in enumerate(cfg.layers):
            pre = f"blocks.{l}."
            attn = {"num_heads": d["heads"], "num_kv_heads": d["kv_heads"], "head_dim": d["head_dim"],
                    "scale": d["head_dim"] ** -0.5, "window": d["window"], "position": PartSpec(*d["position"])}
            layers.append(LayerSpec(f"b{l}", "prenorm_residual",
                                    {"norm_mixer": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, pre + "n1."),
                                     "mixer": PartSpec("gqa_attention", attn, pre + "attn."),
                                     "norm_ffn": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, pre + "n2."),
                                     "ffn": PartSpec(d["ffn"][0], d["ffn"][1], pre + "mlp.")}))
        return ModelSpec("MixedWindowForCausalLM", cfg.width, cfg.vocab_size,
                         PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "emb."), tuple(layers),
                         tuple(range(len(layers))), PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, "norm."),
                         PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": False}, "head."))

    ARCHITECTURES.register("MixedWindowForCausalLM", Architecture("MixedWindowForCausalLM", MixedConfig, spec))


_MIXED_LAYERS = [
    dict(heads=4, kv_heads=2, head_dim=16, window=0, position=("rotary", {"theta": 10000.0, "dim": 16}),
         ffn=("swiglu", {"intermediate_size": 80})),
    dict(heads=4, kv_heads=2, head_dim=16, window=20, position=("rotary", {"theta": 300.0, "dim": 16}),
         ffn=("toy_top1_experts", {"experts": 3, "inner": 24})),
    dict(heads=3, kv_heads=1, head_dim=32, window=9, position=("toy_damped", {"base": 50.0}),
         ffn=("swiglu", {"intermediate_size": 48})),
    dict(heads=4, kv_heads=2, head_dim=16, window=0, position=("none", {}),
         ffn=("toy_top1_experts", {"experts": 2, "inner": 40})),
    # the first layer's theta and width again, after a layer with another theta of the same width: each
    # (theta, width) keeps angles of its own within a step
    dict(heads=4, kv_heads=2, head_dim=16, window=0, position=("rotary", {"theta": 10000.0, "dim": 16}),
         ffn=("swiglu", {"intermediate_size": 64})),
]


def _mixed_plain_logits(raw, t, tokens):
    n, pos = len(tokens), np.arange(len(tokens))
    x = plain.embedding(t["emb.weight"], tokens)
    for l, d in enumerate(raw["layers"]):
        p, nh, nkv, hd = f"blocks.{l}.", d["heads"], d["kv_heads"], d["head_dim"]
        h = plain.rms_norm(x, t[p + "n1.weight"], raw["eps"])
        q = plain.linear(h, t[p + "attn.q_proj.weight"]).reshape(n, nh, hd)
        k = plain.linear(h, t[p + "attn.k_proj.weight"]).reshape(n, nkv, hd)
        v = plain.linear(h, t[p + "attn.v_proj.weight"]).reshape(n, nkv, hd)
        kind, pp = d["position"]
        if kind == "rotary":
            q, k = plain.rotary(q, pos, pp["theta"]), plain.rotary(k, pos, pp["theta"])
        elif kind == "toy_damped":
            f = np.cos(pos[:, None] * np.power(pp["base"], -np.arange(hd) / hd)[None, :])
            q, k = q * f[:, None, :], k * f[:, None, :]
        a = plain.attention(q, k, v, pos, pos, hd ** -0.5, window=d["window"])
        x = x + plain.linear(a.reshape(n, nh * hd), t[p + "attn.o_proj.weight"])
        h = plain.rms_norm(x, t[p + "n2.weight"], raw["eps"])
        if d["ffn"][0] == "swiglu":
            gu = np.concatenate([plain.linear(h, t[p + "mlp.gate_proj.weight"]), plain.linear(h, t[p + "mlp.up_proj.weight"])], -1)
            x = x + plain.linear(plain.swiglu(gu), t[p + "mlp.down_proj.weight"])
        else:
            E, I, H = d["ffn"][1]["experts"], d["ffn"][1]["inner"], raw["width"]
            choice = np.argmax(h @ t[p + "mlp.router.weight"].T, -1)
            w1, w2 = t[p + "mlp.experts.w1"].reshape(E, I, H), t[p + "mlp.experts.w2"].reshape(E, H, I)
            y = np.stack([w2[e] @ np.maximum(w1[e] @ h[r], 0.0) for r, e in enumerate(choice)])
            x = x + y
    return plain.rms_norm(x, t["norm.weight"], raw["eps"]) @ t["head.weight"].T


def test_full_and_windowed_layers_routed_ffn_and_another_position_encoding(tmp_path):
    _register_mixed()
    from kvcm_amd import Engine, EngineConfig
    from kvcm_amd.engine.replay import TraceReplayer
    from kvcm_amd.registry import ARCHITECTURES
    from kvcm_amd.weights.random_init import write_model_dir

    raw = dict(architectures=["MixedWindowForCausalLM"], vocab_size=131, width=56, eps=3e-6, layers=_MIXED_LAYERS)
    cfg = ARCHITECTURES.get("MixedWindowForCausalLM").config_class.from_dict(raw)
    d = write_model_dir(str(tmp_path / "mixed"), "MixedWindowForCausalLM", cfg, seed=21, dtype=torch.float32, std=0.25,
                        norm_jitter=0.1)
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    rng = np.random.default_rng(5)
    reqs = {"a": rng.integers(0, 131, size=90).tolist(), "b": rng.integers(0, 131, size=41).tolist(),
            "c": rng.integers(0, 131, size=57).tolist()}
    ref = {k: _mixed_plain_logits(raw, t, v) for k, v in reqs.items()}

    # 12 pages of 16: a (6 pages) + b (3) + c (4) do not fit together, so c takes pages b gave back
    rp = TraceReplayer(d, "float32", max_tokens=192)
    kinds = [(g.kind, g.window) for g in rp.core.groups]
    assert kinds == [("full", 0), ("window", 20), ("window", 9)]
    assert [[name for name, _ in p.layers] for p in rp.model.groups] == [["b0", "b3", "b4"], ["b1"], ["b2"]]
    steps = [[("a", 0, 30), ("b", 0, 2)], [("a", 30, 33), ("b", 2, 41)], [("a", 33, 34), ("c", 0, 17)],
             [("a", 34, 70), ("c", 17, 18)], [("c", 18, 57)], [("a", 70, 72)]] + [[("a", k, k + 1)] for k in range(72, 90)]
    got = {k: [] for k in reqs}
    for k, entries in enumerate(steps):
        ended = [rid for rid, lo, hi in entries if hi == len(reqs[rid])]
        out = rp.step({"step": k, "entries": [{"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}
                                              for rid, lo, hi in entries], "end": ended})
        row = 0
        for rid, lo, hi in entries:
            got[rid].append(out[row:row + hi - lo])
            row += hi - lo
        if k == 3:
            # a has 70 tokens: the next query (position 70) sees keys from 51 on with window 20, from 62 on with 9
            sid = rp._ids[json.dumps("a")]
            assert [p >= 0 for p in rp.core.seq_table(sid, 0)][:5] == [True] * 5
            assert [p >= 0 for p in rp.core.seq_table(sid, 1)][:5] == [False, False, False, True, True]
            assert [p >= 0 for p in rp.core.seq_table(sid, 2)][:5] == [False, False, False, True, True]
            assert rp.core.blocks_in_use(1) < rp.core.blocks_in_use(0)
    for rid in reqs:
        err = np.abs(np.concatenate(got[rid]) - ref[rid]).max()
        assert err < 1e-4, (rid, err)
    assert all(rp.core.blocks_in_use(g) == 0 for g in range(3))

    # through the scheduler, with few pages and prompts cut into portions
    eng = Engine(d, EngineConfig(dtype="float32", block_size=16, num_blocks=9, max_seq_len=128, max_num_seqs=4,
                                 max_batched_tokens=48, prefill_chunk=13))
    assert eng.decode_graphs is None and eng.model.not_capturable() == ["Damped", "Top1Experts"]
    prompts = [reqs["b"], reqs["c"][:30]]
    outs = eng.generate(prompts, 24)
    for p, g in zip(prompts, outs):
        toks = list(p)
        for k in range(24):
            row = _mixed_plain_logits(raw, t, toks)[-1]
            srt = np.sort(row)
            assert g[k] == int(np.argmax(row)) or srt[-1] - srt[-2] < 1e-4, (k, g[k], int(np.argmax(row)))
            toks.append(g[k])


# ------------------------------------------- another norm and another arrangement of a block
def test_toy_norm_and_parallel_block_arrangement(tmp_path):
    """A norm with mean removal and a bias, and a block that feeds one normed input to mixer and
    feed-forward side by side (x += mixer(n(x)) + ffn(n(x))), both defined here: the norm keeps the
    contract of ``Norm.forward`` (pending addition, row gather), the block that of ``Block.forward``."""
    from kvcm_amd.engine.replay import TraceReplayer
    from kvcm_amd.parts.base import Block, LayerSpec, ModelSpec, Norm, ParamSpec, PartSpec
    from kvcm_amd.registry import ARCHITECTURES, BLOCKS, NORMS, Architecture
    from kvcm_amd.weights.random_init import write_model_dir

    if "toy_layernorm" not in NORMS:
        @NORMS.register("toy_layernorm")
        class ToyLayerNorm(Norm):
            def param_specs(self):
                n = self.params["size"]
                return [ParamSpec("weight", ((self.prefix + "weight", (n,)),), role="vector"),
                        ParamSpec("bias", ((self.prefix + "bias", (n,)),), role="vector")]

            def forward(self, x, out, add=None, rows=None):
                if add is not None:
                    add = add.materialize() if hasattr(add, "materialize") else add
                    if rows is None:
                        x += add.float()
                        v = x
                    else:
                        v = x[rows.long()] + add[rows.long()].float()
                else:
                    v = x if rows is None else x[rows.long()]
                mu = v.mean(-1, keepdim=True)
                var = ((v - mu) ** 2).mean(-1, keepdim=True)
                y = (v - mu) / torch.sqrt(var + self.params["eps"]) * self.w["weight"].float() + self.w["bias"].float()
                out[:v.shape[0]] = y.to(out.dtype)
                return out

        @BLOCKS.register("toy_parallel_residual")
        class ParallelResidual(Block):
            def forward(self, step, x, pending):
                h = step.ws("normed", (step.rows, x.shape[1]))
                self.parts["norm"].forward(x, h, add=pending)                 # adds what the block before left
                a = self.parts["mixer"].forward(step, h)
                a = a.materialize() if hasattr(a, "materialize") else a
                f = self.parts["ffn"].forward(step, h)
                f = f.materialize() if hasattr(f, "materialize") else f
                both = step.ws("both", (step.rows, x.shape[1]), torch.float32)
                both.copy_(a.float() + f.float())
                return both

    @dataclass(frozen=True)
    class Cfg:
        vocab_size: int
        width: int
        heads: int
        head_dim: int
        inner: int
        depth: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("vocab_size", "width", "heads", "head_dim", "inner", "depth", "eps")})

        def to_dict(self):
            return asdict(self)

    def spec(cfg):
        def norm(prefix):
            return PartSpec("toy_layernorm", {"size": cfg.width, "eps": cfg.eps}, prefix)
        attn = {"num_heads": cfg.heads, "num_kv_heads": cfg.heads, "head_dim": cfg.head_dim, "scale": cfg.head_dim ** -0.5,
                "window": 0, "position": PartSpec("rotary", {"theta": 1000.0, "dim": cfg.head_dim})}
        layers = tuple(LayerSpec(f"p{l}", "toy_parallel_residual",
                                 {"norm": norm(f"h.{l}.ln."), "mixer": PartSpec("gqa_attention", attn, f"h.{l}.attn."),
                                  "ffn": PartSpec("swiglu", {"intermediate_size": cfg.inner}, f"h.{l}.mlp.")})
                       for l in range(cfg.depth))
        return ModelSpec("ToyParallelForCausalLM", cfg.width, cfg.vocab_size,
                         PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "wte."), layers, tuple(range(cfg.depth)),
                         norm("ln_f."), PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": True}, "head."))

    ARCHITECTURES.register("ToyParallelForCausalLM", Architecture("ToyParallelForCausalLM", Cfg, spec))
    raw = dict(architectures=["ToyParallelForCausalLM"], vocab_size=77, width=40, heads=2, head_dim=16, inner=72, depth=2, eps=2e-5)
    cfg = Cfg.from_dict(raw)
    d = write_model_dir(str(tmp_path / "par"), "ToyParallelForCausalLM", cfg, seed=13, dtype=torch.float32, std=0.2, norm_jitter=0.2)
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    toks = np.random.default_rng(2).integers(0, 77, size=41).tolist()

    def ln(v, pre):
        mu = v.mean(-1, keepdims=True)
        var = ((v - mu) ** 2).mean(-1, keepdims=True)
        return (v - mu) / np.sqrt(var + raw["eps"]) * t[pre + "weight"] + t[pre + "bias"]

    n, pos = len(toks), np.arange(len(toks))
    x = plain.embedding(t["wte.weight"], toks)
    for l in range(2):
        p = f"h.{l}."
        h = ln(x, p + "ln.")
        q = plain.rotary(plain.linear(h, t[p + "attn.q_proj.weight"]).reshape(n, 2, 16), pos, 1000.0)
        k = plain.rotary(plain.linear(h, t[p + "attn.k_proj.weight"]).reshape(n, 2, 16), pos, 1000.0)
        v = plain.linear(h, t[p + "attn.v_proj.weight"]).reshape(n, 2, 16)
        a = plain.linear(plain.attention(q, k, v, pos, pos, 0.25).reshape(n, 32), t[p + "attn.o_proj.weight"])
        gu = np.concatenate([plain.linear(h, t[p + "mlp.gate_proj.weight"]), plain.linear(h, t[p + "mlp.up_proj.weight"])], -1)
        x = x + a + plain.linear(plain.swiglu(gu), t[p + "mlp.down_proj.weight"])
    ref = ln(x, "ln_f.") @ t["wte.weight"].T

    rp = TraceReplayer(d, "float32", max_tokens=64)
    a = rp.step({"step": 0, "entries": [{"id": "s", "tokens": toks[:17], "want": list(range(17))}], "end": []})
    b = rp.step({"step": 1, "entries": [{"id": "s", "tokens": toks[17:19], "want": [0, 1]}], "end": []})
    c = rp.step({"step": 2, "entries": [{"id": "s", "tokens": toks[19:], "want": list(range(22))}], "end": ["s"]})
    np.testing.assert_allclose(np.concatenate([a, b, c]), ref, atol=2e-4)


# ----------------------------------------- two cache owners in one layer, under names of their own
def test_a_layer_with_an_attention_and_a_state_mixer_side_by_side(tmp_path):
    """A block arrangement defined here holds two parts that each keep something per request: an attention
    over paged keys and values ("look") and the toy mixer with a state slot ("remember"); a second layer of
    the same kind whose attention reads the first layer's pages.  Both get their caches from the model's
    planner (one paged group, one state group), are stepped in portions beside other requests with pages
    used again, and equal a plain toy."""
    _register_toy()
    from kvcm_amd.engine.replay import TraceReplayer
    from kvcm_amd.parts.base import Block, LayerSpec, ModelSpec, PartSpec, as_tensor
    from kvcm_amd.registry import ARCHITECTURES, BLOCKS, Architecture
    from kvcm_amd.weights.random_init import write_model_dir

    if "toy_two_memories" not in BLOCKS:
        @BLOCKS.register("toy_two_memories")
        class TwoMemories(Block):
            """x += look(n(x)) + remember(n(x)); x += ffn(n2(x))."""
            part_registries = {"look": "mixer", "remember": "mixer"}

            def forward(self, step, x, pending):
                h = step.ws("normed", (step.rows, x.shape[1]))
                self.parts["norm_in"].forward(x, h, add=as_tensor(pending))
                both = step.ws("both", (step.rows, x.shape[1]), torch.float32)
                both.copy_(as_tensor(self.parts["look"].forward(step, h)).float())     # (the two mixers use one work buffer)
                both += self.parts["remember"].forward(step, h).float()
                self.parts["norm_ffn"].forward(x, h, add=both)
                return as_tensor(self.parts["ffn"].forward(step, h))

    @dataclass(frozen=True)
    class Cfg:
        vocab_size: int
        width: int
        heads: int
        kv_heads: int
        head_dim: int
        inner: int
        state_size: int
        decay: float
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("vocab_size", "width", "heads", "kv_heads", "head_dim", "inner", "state_size",
                                              "decay", "eps")})

        def to_dict(self):
            return asdict(self)

    def spec(cfg):
        def layer(name, prefix, cache_from=None):
            attn = {"num_heads": cfg.heads, "num_kv_heads": cfg.kv_heads, "head_dim": cfg.head_dim, "scale": cfg.head_dim ** -0.5,
                    "window": 0, "position": PartSpec("rotary", {"theta": 5000.0, "dim": cfg.head_dim})}
            return LayerSpec(name, "toy_two_memories", {
                "norm_in": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix + "n1."),
                "look": PartSpec("gqa_attention", attn, prefix + "attn."),
                "remember": PartSpec("toy_decay_state", {"state_size": cfg.state_size, "decay": cfg.decay}, prefix + "mix."),
                "norm_ffn": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix + "n2."),
                "ffn": PartSpec("swiglu", {"intermediate_size": cfg.inner}, prefix + "mlp.")}, cache_from)
        # the second layer's attention reads the first layer's keys and values; its state mixer keeps a state of its own
        layers = (layer("first", "l0."), layer("second", "l1.", {"look": "first.look"}))
        return ModelSpec("ToyTwoMemoriesForCausalLM", cfg.width, cfg.vocab_size,
                         PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "emb."), layers, (0, 1),
                         PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, "out_norm."),
                         PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": True}, "head."))

    ARCHITECTURES.register("ToyTwoMemoriesForCausalLM", Architecture("ToyTwoMemoriesForCausalLM", Cfg, spec))
    raw = dict(architectures=["ToyTwoMemoriesForCausalLM"], vocab_size=83, width=48, heads=4, kv_heads=2, head_dim=16, inner=64,
               state_size=12, decay=0.8, eps=1e-5)
    cfg = Cfg.from_dict(raw)
    d = write_model_dir(str(tmp_path / "two"), "ToyTwoMemoriesForCausalLM", cfg, seed=21, dtype=torch.float32, std=0.25, norm_jitter=0.1)
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    # (the second layer's attention has no k and v projections of its own to read: the loader asks for them all the same,
    # they are simply not used for the cache it reads)

    def plain_logits(tokens):
        n, pos = len(tokens), np.arange(len(tokens))
        x = plain.embedding(t["emb.weight"], tokens)
        first_kv = None
        for l, p in enumerate(("l0.", "l1.")):
            h = plain.rms_norm(x, t[p + "n1.weight"], raw["eps"])
            q = plain.rotary(plain.linear(h, t[p + "attn.q_proj.weight"]).reshape(n, 4, 16), pos, 5000.0)
            if l == 0:
                k = plain.rotary(plain.linear(h, t[p + "attn.k_proj.weight"]).reshape(n, 2, 16), pos, 5000.0)
                v = plain.linear(h, t[p + "attn.v_proj.weight"]).reshape(n, 2, 16)
                first_kv = (k, v)
            k, v = first_kv
            a = plain.linear(plain.attention(q, k, v, pos, pos, 0.25).reshape(n, 64), t[p + "attn.o_proj.weight"])
            u = h @ t[p + "mix.in_proj.weight"].T
            state, b = np.zeros(raw["state_size"]), np.zeros_like(x)
            for r in range(n):
                state = raw["decay"] * state + u[r]
                b[r] = t[p + "mix.out_proj.weight"] @ state
            x = x + a + b
            h = plain.rms_norm(x, t[p + "n2.weight"], raw["eps"])
            gu = np.concatenate([plain.linear(h, t[p + "mlp.gate_proj.weight"]), plain.linear(h, t[p + "mlp.up_proj.weight"])], -1)
            x = x + plain.linear(plain.swiglu(gu), t[p + "mlp.down_proj.weight"])
        return plain.rms_norm(x, t["out_norm.weight"], raw["eps"]) @ t["emb.weight"].T

    rng = np.random.default_rng(8)
    reqs = {"x": rng.integers(0, 83, size=37).tolist(), "y": rng.integers(0, 83, size=9).tolist(),
            "z": rng.integers(0, 83, size=50).tolist(), "w": rng.integers(0, 83, size=21).tolist()}
    ref = {k: plain_logits(v) for k, v in reqs.items()}
    rp = TraceReplayer(d, "float32", max_tokens=128, max_live=3)         # 8 pages: x, y and z fill them, w runs on pages given back
    assert [(g.kind, [name for name, _ in plan.layers]) for g, plan in zip(rp.core.groups, rp.model.groups)] == \
        [("full", ["first"]), ("state", ["first", "second"])]
    assert [part for _, part in rp.model.groups[0].layers] == ["look"] and [part for _, part in rp.model.groups[1].layers] == ["remember"] * 2
    steps = [[("x", 0, 11), ("y", 0, 2)], [("x", 11, 12), ("y", 2, 9), ("z", 0, 30)], [("x", 12, 37), ("z", 30, 31)],
             [("z", 31, 50), ("w", 0, 3)], [("w", 3, 21)]]
    got = {k: [] for k in reqs}
    for k, entries in enumerate(steps):
        ended = [rid for rid, lo, hi in entries if hi == len(reqs[rid])]
        out = rp.step({"step": k, "entries": [{"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}
                                              for rid, lo, hi in entries], "end": ended})
        row = 0
        for rid, lo, hi in entries:
            got[rid].append(out[row:row + hi - lo])
            row += hi - lo
    for rid in reqs:
        err = np.abs(np.concatenate(got[rid]) - ref[rid]).max()
        assert err < 2e-4, (rid, err)
    assert rp.core.blocks_in_use(0) == 0 and rp.core.state_slots_free() == 3
