"""Configuration reading, the registry, weight checking and the random-weights mode (no GPU)."""
import json
import os

import numpy as np
import pytest
import torch

import helpers as H
import plain_llama as plain
from kvcm_amd import architectures  # noqa: F401
from kvcm_amd.config.engine_config import EngineConfig
from kvcm_amd.config.model_config import ConfigError, LlamaConfig, read_config_json
from kvcm_amd.parts.base import BuildContext, KVCacheNeed
from kvcm_amd.parts.model import Model
from kvcm_amd.registry import ARCHITECTURES, MIXERS
from kvcm_amd.weights.loader import DictSource, FolderSource, WeightsError, check_against, load_weights
from kvcm_amd.weights.random_init import expected_tensors, random_tensors, write_model_dir
from kvcm_amd.weights.safetensors_io import SafetensorsFile, write_safetensors


def _model(raw, dtype=torch.float32):
    cfg = LlamaConfig.from_dict(raw)
    spec = ARCHITECTURES.get("LlamaForCausalLM").build_spec(cfg)
    return cfg, Model(spec, BuildContext(dtype, torch.device("cpu"), spec.hidden_size, 16, None))


# ---------------------------------------------------------------------- seeded random weights
def test_random_weights_follow_the_counter_rule_of_the_plain_implementation():
    """The engine's host generator and the plain implementation's, written apart from each other from
    the same rule, give the same bits; the values are normal; a tensor depends on (seed, name) alone."""
    from kvcm_amd.weights.random_init import normal_values, random_tensor, tensor_key
    for seed, name, count in ((0, "model.embed_tokens.weight", 100003), (7, "model.layers.3.mlp.up_proj.weight", 4097),
                              ((1 << 63) + 5, "x", 1)):
        got = normal_values(tensor_key(seed, name), count)
        want = plain.counter_normal(seed, name, count)
        assert got.dtype == np.float32 and np.array_equal(got, want)
    big = normal_values(tensor_key(0, "model.embed_tokens.weight"), 400000, chunk=65536)       # chunking changes nothing
    np.testing.assert_array_equal(big[:100003], plain.counter_normal(0, "model.embed_tokens.weight", 100003))
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1) < 0.01 and abs((big ** 3).mean()) < 0.03
    assert abs((big ** 4).mean() - 3) < 0.1 and 4 < np.abs(big).max() < 7
    # the same tensor whatever else was made before it, another one for another name or seed
    a = random_tensor(3, "w.weight", (50, 20), "matrix", torch.float32)
    np.testing.assert_array_equal(a.numpy(), plain.counter_weight(3, "w.weight", (50, 20)))
    assert not np.array_equal(a.numpy(), plain.counter_weight(3, "v.weight", (50, 20)))
    assert not np.array_equal(a.numpy(), plain.counter_weight(4, "w.weight", (50, 20)))
    g = random_tensor(3, "n.weight", (64,), "vector", torch.float32, norm_jitter=0.1)
    np.testing.assert_array_equal(g.numpy(), plain.counter_weight(3, "n.weight", (64,), vector=True, norm_jitter=0.1))
    assert torch.equal(random_tensor(3, "n.weight", (64,), "vector", torch.float32), torch.ones(64))
    idx = random_tensor(3, "table", (1000,), "index")
    assert idx.dtype == torch.int32 and 0 <= int(idx.min()) and int(idx.max()) < 1024 and len(set(idx.tolist())) > 500
    # bfloat16 storage is the float32 value rounded
    b = random_tensor(3, "w.weight", (50, 20), "matrix", torch.bfloat16)
    np.testing.assert_array_equal(b.float().numpy(), plain.round_bf16(a.numpy()).astype(np.float32))


# ------------------------------------------------------------------------------------ config
def test_config_reads_its_keys_and_defaults():
    c = LlamaConfig.from_dict(H.TINY_A)
    assert (c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (256, 64, 176, 2)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (4, 2, 16)
    assert c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-5 and not c.tie_word_embeddings
    assert (c.q_dim, c.kv_dim, c.qkv_dim) == (64, 32, 128)
    assert c.num_parameters() == 125248
    assert LlamaConfig.from_dict(H.TINY_B).num_parameters() == 332448
    minimal = dict(vocab_size=10, hidden_size=24, intermediate_size=20, num_hidden_layers=1, num_attention_heads=3)
    m = LlamaConfig.from_dict(minimal)
    assert m.num_key_value_heads == 3 and m.head_dim == 8                  # defaults derived
    assert m.rope_theta == 10000.0 and m.rms_norm_eps == 1e-5 and m.max_position_embeddings == 2048
    # head_dim may differ from hidden/heads
    assert LlamaConfig.from_dict(H.TINY_C).head_dim == 48
    # TinyLlama-1.1B sizes
    big = dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
               num_attention_heads=32, num_key_value_heads=4)
    assert LlamaConfig.from_dict(big).num_parameters() == 1100048384


@pytest.mark.parametrize("patch,fragment", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"head_dim": 15}, "head_dim 15 is not supported"),
    ({"head_dim": 12}, "multiples of 8 up to 256"),           # even, but not what the kernels take
    ({"head_dim": 264}, "head_dim 264"),
    ({"hidden_size": 40, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": None}, "head_dim 10"),       # derived
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "rope_scaling"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"hidden_size": "64"}, "hidden_size"),
    ({"rms_norm_eps": 0}, "rms_norm_eps"),
])
def test_config_refuses_what_the_engine_has_not(patch, fragment):
    with pytest.raises(ConfigError, match=fragment):
        LlamaConfig.from_dict({**H.TINY_A, **patch})


def test_config_takes_rope_scaling_that_says_no_scaling():
    for value in (None, {}, {"rope_type": "default"}, {"type": "default"}):
        assert LlamaConfig.from_dict({**H.TINY_A, "rope_scaling": value}).rope_theta == H.TINY_A.get("rope_theta", 10000.0)
    with pytest.raises(ConfigError, match="rope_scaling"):
        LlamaConfig.from_dict({**H.TINY_A, "rope_scaling": {"rope_type": "llama3", "factor": 8.0}})


def test_config_lists_every_problem_at_once():
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict({**H.TINY_A, "head_dim": 7, "attention_bias": True, "hidden_act": "relu"})
    msg = str(e.value)
    assert "head_dim" in msg and "attention_bias" in msg and "hidden_act" in msg


def test_architecture_comes_from_config_json(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(H.TINY_A))
    name, raw = read_config_json(str(tmp_path))
    assert name == "LlamaForCausalLM" and raw["hidden_size"] == 64
    with pytest.raises(KeyError, match="registered.*LlamaForCausalLM"):
        ARCHITECTURES.get("SomethingElseForCausalLM")
    (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in H.TINY_A.items() if k != "architectures"}))
    with pytest.raises(ConfigError, match="architectures"):
        read_config_json(str(tmp_path))
    with pytest.raises(ConfigError, match="no config.json"):
        read_config_json(str(tmp_path / "nowhere"))


def test_engine_config_validation():
    assert EngineConfig().validate().max_num_seqs == 256 and EngineConfig().max_batched_tokens == 4096
    with pytest.raises(ValueError, match="policy"):
        EngineConfig(policy="buddy").validate()
    with pytest.raises(ValueError, match="attention version"):
        EngineConfig(attn="v3").validate()
    with pytest.raises(ValueError, match="dtype"):
        EngineConfig(dtype="fp8").validate()


# --------------------------------------------------------------------- the model as data
def test_llama_spec_is_data_over_registered_parts():
    cfg, model = _model(H.TINY_B)
    spec = model.spec
    assert len(spec.layers) == 3 and spec.schedule == (0, 1, 2)
    mixer = spec.layers[1].parts["mixer"]
    assert mixer.kind == "gqa_attention" and mixer.kind in MIXERS
    assert mixer.params["num_heads"] == 3 and mixer.params["num_kv_heads"] == 1 and mixer.params["head_dim"] == 32
    assert mixer.params["position"].params == {"theta": 500000.0, "dim": 32}
    assert spec.layers[0].parts["norm_ffn"].params == {"size": 96, "eps": 1e-6}
    assert spec.head.params["tied"] is True
    assert len(model.groups) == 1 and model.groups[0].need == KVCacheNeed(1, 32, 0)
    assert model.groups[0].layers == [("layers.0", "mixer"), ("layers.1", "mixer"), ("layers.2", "mixer")]


def test_expected_tensor_names_follow_the_checkpoint_layout():
    names = expected_tensors("LlamaForCausalLM", LlamaConfig.from_dict(H.TINY_A))
    assert names["model.embed_tokens.weight"] == ((256, 64), "table")
    assert names["model.layers.1.self_attn.k_proj.weight"] == ((32, 64), "matrix")
    assert names["model.layers.0.mlp.down_proj.weight"] == ((64, 176), "matrix")
    assert names["model.layers.0.post_attention_layernorm.weight"] == ((64,), "vector")
    assert names["lm_head.weight"] == ((256, 64), "table") and names["model.norm.weight"] == ((64,), "vector")
    assert len(names) == 3 + 9 * 2
    tied = expected_tensors("LlamaForCausalLM", LlamaConfig.from_dict(H.TINY_B))
    assert "lm_head.weight" not in tied and len(tied) == 2 + 9 * 3


# ----------------------------------------------------------------------------------- weights
def test_random_weights_folder_round_trips(tmp_path):
    cfg = LlamaConfig.from_dict(H.TINY_A)
    d = write_model_dir(str(tmp_path / "m"), "LlamaForCausalLM", cfg, seed=3, dtype=torch.bfloat16)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    arch, raw = read_config_json(d)
    assert arch == "LlamaForCausalLM" and LlamaConfig.from_dict(raw) == cfg
    src = FolderSource(d)
    again = random_tensors("LlamaForCausalLM", cfg, seed=3, dtype=torch.bfloat16)
    other = random_tensors("LlamaForCausalLM", cfg, seed=4, dtype=torch.bfloat16)
    for n in src.names():
        assert src.dtype(n) == torch.bfloat16
        assert torch.equal(src.get(n), again[n]), "same seed, same tensors, whatever the order"
    assert not torch.equal(again["lm_head.weight"], other["lm_head.weight"])
    w = again["model.layers.0.mlp.up_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    assert torch.equal(again["model.norm.weight"], torch.ones(64, dtype=torch.bfloat16))
    # the plain reader sees the same numbers
    pt = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    np.testing.assert_array_equal(pt["lm_head.weight"], again["lm_head.weight"].float().numpy())
    src.close()


def test_loader_fuses_by_name_and_keeps_precisions(tmp_path):
    cfg, model = _model(H.TINY_A, torch.bfloat16)
    tensors = random_tensors("LlamaForCausalLM", cfg, seed=1, dtype=torch.bfloat16)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float() * 1.0001      # stored in 32 bits
    load_weights(model, DictSource(tensors), torch.bfloat16, "cpu")
    mixer = model.layer_parts[0]["mixer"]
    q, k, v = (tensors[f"model.layers.0.self_attn.{n}_proj.weight"] for n in "qkv")
    assert torch.equal(mixer.w["wqkv"], torch.cat([q, k, v], 0)) and mixer.w["wqkv"].dtype == torch.bfloat16
    ffn = model.layer_parts[1]["ffn"]
    assert torch.equal(ffn.w["w_gate_up"], torch.cat([tensors["model.layers.1.mlp.gate_proj.weight"],
                                                      tensors["model.layers.1.mlp.up_proj.weight"]], 0))
    assert model.final_norm.w["weight"].dtype == torch.float32                        # a 32-bit vector stays 32-bit
    assert model.layer_parts[0]["norm_mixer"].w["weight"].dtype == torch.bfloat16
    # the 32-bit path widens everything
    cfg, model32 = _model(H.TINY_A, torch.float32)
    load_weights(model32, DictSource(tensors), torch.float32, "cpu")
    assert all(t.dtype == torch.float32 for p in model32.all_parts() for t in p.w.values())
    assert torch.equal(model32.head.w["table"], tensors["lm_head.weight"].float())


def test_tied_head_shares_the_embedding_table():
    cfg, model = _model(H.TINY_B)
    tensors = random_tensors("LlamaForCausalLM", cfg, seed=2, dtype=torch.float32)
    load_weights(model, DictSource(tensors), torch.float32, "cpu")
    assert model.head.w["table"] is model.embedding.w["table"]
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()          # a stored copy is tolerated
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)          # so is a derived buffer
    check_against(model, DictSource(tensors))


def test_one_error_lists_missing_unexpected_and_misshapen():
    cfg, model = _model(H.TINY_A)
    t = random_tensors("LlamaForCausalLM", cfg, seed=1, dtype=torch.float32)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    t["model.layers.0.mlp.down_proj.weight"] = torch.zeros(64, 175)
    t["model.embed_tokens.weight"] = torch.zeros(255, 64)
    with pytest.raises(WeightsError) as e:
        load_weights(model, DictSource(t), torch.float32, "cpu")
    msg = str(e.value)
    assert "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.q_proj.bias" in msg
    assert "wrong shapes (2)" in msg and "model.embed_tokens.weight expected [256, 64] got [255, 64]" in msg
    assert "model.layers.0.mlp.down_proj.weight expected [64, 176] got [64, 175]" in msg


def test_safetensors_files_are_checked(tmp_path):
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.ones(4, dtype=torch.bfloat16),
                          "c": torch.arange(5, dtype=torch.int32)})
    f = SafetensorsFile(p)
    assert f.shape("a") == (2, 3) and f.dtype("b") == torch.bfloat16 and f.dtype("c") == torch.int32
    assert torch.equal(f.tensor("a"), torch.arange(6, dtype=torch.float32).reshape(2, 3))
    assert torch.equal(f.tensor("b"), torch.ones(4, dtype=torch.bfloat16))
    f.close()
    raw = open(p, "rb").read()
    open(p, "wb").write(raw[:-3])
    with pytest.raises(ValueError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(b"\x05")
    with pytest.raises(ValueError, match="too short"):
        SafetensorsFile(p)
    os.makedirs(str(tmp_path / "empty"))
    with pytest.raises(WeightsError, match="no model.safetensors"):
        FolderSource(str(tmp_path / "empty"))


# ---------------------------------------------------------------- the plain implementation
def test_plain_rms_norm_pins():
    x = np.full((1, 64), 0.01)
    np.testing.assert_allclose(plain.rms_norm(x, np.ones(64), 1e-4), 0.01 / np.sqrt(1e-4 + 1e-4))   # eps inside the root
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 50))
    w = rng.normal(size=50)
    np.testing.assert_allclose(plain.rms_norm(x, w, 1e-6), x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-6) * w)
    np.testing.assert_allclose(plain.rms_norm(1000 * x, w, 1e-6), plain.rms_norm(x, w, 1e-6), rtol=1e-6)  # scale-free
    m = x + 5.0
    assert not np.allclose(plain.rms_norm(m, w, 1e-6), plain.rms_norm(m - m.mean(-1, keepdims=True), w, 1e-6))  # no mean removed


def test_plain_rotary_pins():
    rng = np.random.default_rng(1)
    v = rng.normal(size=(4, 2, 16))
    pos = np.array([0, 1, 7, 100])
    r = plain.rotary(v, pos, 10000.0)
    np.testing.assert_array_equal(r[0], v[0])                                    # position 0 is the identity
    np.testing.assert_allclose(r[..., :8] ** 2 + r[..., 8:] ** 2, v[..., :8] ** 2 + v[..., 8:] ** 2)  # pair lengths
    # a complex multiplication of (v[j] + i v[j + hd/2]) by exp(i * pos * theta^(-2j/hd))
    j = np.arange(8)
    ang = pos[:, None] * 10000.0 ** (-2.0 * j / 16)
    z = (v[..., :8] + 1j * v[..., 8:]) * np.exp(1j * ang)[:, None, :]
    np.testing.assert_allclose(r[..., :8], z.real, atol=1e-5)
    np.testing.assert_allclose(r[..., 8:], z.imag, atol=1e-5)
    # an interleaved pairing (2j, 2j+1) would fail this: the first pair is (0, 8), not (0, 1)
    e = np.zeros((1, 1, 16))
    e[0, 0, 0] = 1.0
    out = plain.rotary(e, [1], 10000.0)[0, 0]
    assert abs(out[8] - np.sin(1.0)) < 1e-6 and abs(out[1]) < 1e-12
    # scores depend on the distance only
    q, k = rng.normal(size=(1, 1, 16)), rng.normal(size=(1, 1, 16))
    d = lambda a, b: float((plain.rotary(q, [a], 1e4) * plain.rotary(k, [b], 1e4)).sum())
    assert abs(d(9, 4) - d(109, 104)) < 1e-4 and abs(d(9, 4) - d(9, 5)) > 1e-3


def test_plain_attention_pins():
    rng = np.random.default_rng(2)
    q, k, v = rng.normal(size=(5, 4, 8)), rng.normal(size=(5, 2, 8)), rng.normal(size=(5, 2, 8))
    pos = np.arange(5)
    out = plain.attention(q, k, v, pos, pos, 8 ** -0.5)
    np.testing.assert_allclose(out[0], v[0][[0, 0, 1, 1]])                       # one key: its value, head h -> kv head h // 2
    tq, tk, tv = torch.tensor(q).permute(1, 0, 2)[None], torch.tensor(k).permute(1, 0, 2), torch.tensor(v).permute(1, 0, 2)
    lib = torch.nn.functional.scaled_dot_product_attention(tq, tk.repeat_interleave(2, 0)[None], tv.repeat_interleave(2, 0)[None],
                                                           is_causal=True)[0].permute(1, 0, 2).numpy()
    np.testing.assert_allclose(out, lib, atol=1e-12)
    same = plain.attention(q, np.ones_like(k), v, pos, pos, 1.0)
    np.testing.assert_allclose(same[4, 0], v[:, 0].mean(0))                      # equal keys: the mean of the values
    win = plain.attention(q, k, v, pos, pos, 1.0, window=2)
    np.testing.assert_allclose(win[4], plain.attention(q[4:], k[3:], v[3:], [4], [3, 4], 1.0)[0])


def test_plain_swiglu_and_sampling_pins():
    gu = np.array([[0.0, 30.0, -30.0, 1.0, 2.0, 3.0, 4.0, 5.0]])
    np.testing.assert_allclose(plain.swiglu(gu), [[0.0, 30.0 * 3.0, 0.0, 1 / (1 + np.exp(-1.0)) * 5.0]], atol=1e-10)
    assert plain.argmax_rows(np.array([[1.0, 5.0, 5.0, 2.0]]))[0] == 1           # lowest index among equal maxima
    logits = np.log(np.array([0.1, 0.2, 0.3, 0.4]))
    draws = [plain.sample_row(logits, 1.0, seed, 0, 0)[0] for seed in range(3000)]
    np.testing.assert_allclose(np.bincount(draws, minlength=4) / 3000.0, [0.1, 0.2, 0.3, 0.4], atol=0.03)
    assert plain.sample_row(logits, 1e-4, 5, 0, 0)[0] == 3                       # temperature -> 0 is the argmax
    assert plain.sample_row(logits, 1.0, 5, 1, 2) == plain.sample_row(logits, 1.0, 5, 1, 2)
    np.testing.assert_array_equal(plain.round_bf16(np.array([1.0, 1.00390625, 1.01171875, 3.14159])),
                                  [1.0, 1.0, 1.015625, 3.140625])                # ties to even


def _tiny_plain(seed=0, **zeroed):
    raw = H.TINY_A
    t = {k: v.numpy().astype(np.float64) for k, v in
         random_tensors("LlamaForCausalLM", LlamaConfig.from_dict(raw), seed=seed, dtype=torch.float32, std=0.2, norm_jitter=0.2).items()}
    for name in t:
        if any(name.endswith(z) for z in zeroed.get("zero", ())):
            t[name] = np.zeros_like(t[name])
    return raw, t, plain.PlainLlama(raw, t)


def test_plain_model_residual_placement_and_layer_order():
    """What the layers add to the residual stream, where the norms sit and in which order the two
    halves of a layer run, pinned by cases that reduce to something smaller (src/model/llama.cpp:104-128)."""
    toks = list(np.random.default_rng(4).integers(0, 256, size=9))
    pos = np.arange(9)
    # nothing but the residual path: both output projections zero -> head(final_norm(embedding))
    raw, t, pm = _tiny_plain(zero=("o_proj.weight", "down_proj.weight"))
    emb = plain.embedding(t["model.embed_tokens.weight"], toks)
    bare = plain.rms_norm(emb, t["model.norm.weight"], raw["rms_norm_eps"]) @ t["lm_head.weight"].T
    np.testing.assert_allclose(pm.logits(toks), bare, atol=1e-12)
    # ... and the final norm is applied to the stream itself: a larger embedding changes nothing
    t10 = dict(t)
    t10["model.embed_tokens.weight"] = t["model.embed_tokens.weight"] * 1000.0
    np.testing.assert_allclose(plain.PlainLlama(raw, t10).logits(toks), bare, rtol=1e-3, atol=1e-6)   # (eps is what is left)

    # attention alone: down_proj zero -> x += o(attn(rot(q), rot(k), v)) of norm1(x), layer after layer
    raw, t, pm = _tiny_plain(zero=("down_proj.weight",))
    x = plain.embedding(t["model.embed_tokens.weight"], toks)
    for l in range(raw["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = plain.rms_norm(x, t[p + "input_layernorm.weight"], raw["rms_norm_eps"])
        q = plain.rotary(plain.linear(h, t[p + "self_attn.q_proj.weight"]).reshape(9, 4, 16), pos, raw["rope_theta"])
        k = plain.rotary(plain.linear(h, t[p + "self_attn.k_proj.weight"]).reshape(9, 2, 16), pos, raw["rope_theta"])
        v = plain.linear(h, t[p + "self_attn.v_proj.weight"]).reshape(9, 2, 16)
        x = x + plain.linear(plain.attention(q, k, v, pos, pos, 0.25).reshape(9, 64), t[p + "self_attn.o_proj.weight"])
    want = plain.rms_norm(x, t["model.norm.weight"], raw["rms_norm_eps"]) @ t["lm_head.weight"].T
    np.testing.assert_allclose(pm.logits(toks), want, atol=1e-10)
    # a post-norm arrangement (norm after the addition) or an un-normed input to q/k/v would differ
    post = plain.embedding(t["model.embed_tokens.weight"], toks)
    for l in range(raw["num_hidden_layers"]):
        p = f"model.layers.{l}."
        q = plain.rotary(plain.linear(post, t[p + "self_attn.q_proj.weight"]).reshape(9, 4, 16), pos, raw["rope_theta"])
        k = plain.rotary(plain.linear(post, t[p + "self_attn.k_proj.weight"]).reshape(9, 2, 16), pos, raw["rope_theta"])
        v = plain.linear(post, t[p + "self_attn.v_proj.weight"]).reshape(9, 2, 16)
        a = plain.linear(plain.attention(q, k, v, pos, pos, 0.25).reshape(9, 64), t[p + "self_attn.o_proj.weight"])
        post = plain.rms_norm(post + a, t[p + "input_layernorm.weight"], raw["rms_norm_eps"])
    assert np.abs(post - x).max() > 1e-2

    # the feed-forward alone: o_proj zero -> rows do not see each other at all, and every layer adds
    # down(swiglu(gate(h), up(h))) of norm2(x); a position's logits depend on its own token only
    raw, t, pm = _tiny_plain(zero=("o_proj.weight",))
    x = plain.embedding(t["model.embed_tokens.weight"], toks)
    for l in range(raw["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = plain.rms_norm(x, t[p + "post_attention_layernorm.weight"], raw["rms_norm_eps"])
        gu = np.concatenate([plain.linear(h, t[p + "mlp.gate_proj.weight"]), plain.linear(h, t[p + "mlp.up_proj.weight"])], -1)
        x = x + plain.linear(plain.swiglu(gu), t[p + "mlp.down_proj.weight"])
    want = plain.rms_norm(x, t["model.norm.weight"], raw["rms_norm_eps"]) @ t["lm_head.weight"].T
    np.testing.assert_allclose(pm.logits(toks), want, atol=1e-10)
    np.testing.assert_allclose(pm.logits(toks[3:4])[0], pm.logits(toks)[3], atol=1e-10)

    # order inside a layer: the feed-forward reads the stream after the attention's addition.  With the
    # first layer's attention swapped for another one the feed-forward's input changes, so its own
    # contribution (its output for the same tokens) changes too; side by side on one input it would not.
    raw, t, pm = _tiny_plain()
    full = pm.logits(toks)
    t2 = dict(t)
    t2["model.layers.0.self_attn.o_proj.weight"] = -t["model.layers.0.self_attn.o_proj.weight"]
    x_a = plain.PlainLlama(raw, t).layer(0, plain.embedding(t["model.embed_tokens.weight"], toks), pos)
    x_b = plain.PlainLlama(raw, t2).layer(0, plain.embedding(t["model.embed_tokens.weight"], toks), pos)
    emb = plain.embedding(t["model.embed_tokens.weight"], toks)
    h = plain.rms_norm(emb, t["model.layers.0.input_layernorm.weight"], raw["rms_norm_eps"])
    q = plain.rotary(plain.linear(h, t["model.layers.0.self_attn.q_proj.weight"]).reshape(9, 4, 16), pos, raw["rope_theta"])
    k = plain.rotary(plain.linear(h, t["model.layers.0.self_attn.k_proj.weight"]).reshape(9, 2, 16), pos, raw["rope_theta"])
    v = plain.linear(h, t["model.layers.0.self_attn.v_proj.weight"]).reshape(9, 2, 16)
    a = plain.linear(plain.attention(q, k, v, pos, pos, 0.25).reshape(9, 64), t["model.layers.0.self_attn.o_proj.weight"])
    ffn_a, ffn_b = x_a - (emb + a), x_b - (emb - a)          # what the feed-forward added in each case
    assert np.abs(ffn_a - ffn_b).max() > 1e-3                # it saw the attention's output
    assert full.shape == (9, 256)


def test_plain_rounding_positions_on_the_16_bit_grid():
    """The two places where the order of rounding and multiplying matters (src/cuda/kernels.cu:34-49:
    the normed value is cast to 16 bits, then multiplied by the weight in 16 bits; kernels.cu:72-82:
    silu is cast to 16 bits, then multiplied by up), with inputs on which another order gives other bits."""
    r = plain.round_bf16
    x, w = H.norm_rounding_cases()
    inv = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
    ours = plain.rms_norm(x, w, 1e-6, r)
    np.testing.assert_array_equal(ours, r(w * r(x * inv)))
    assert (ours != r(w * x * inv)).mean() > 0.05            # rounding once, after the multiply
    assert (ours != r(r(w * x) * inv)).mean() > 0.05         # weight first
    g, u = H.swiglu_rounding_cases()
    act = plain.swiglu(np.concatenate([g, u], -1), r)
    silu = g / (1.0 + np.exp(-g))
    np.testing.assert_array_equal(act, r(r(silu) * u))
    assert (act != r(silu * u)).mean() > 0.05                # rounding once, after the multiply
    assert (act != r(g * r(1.0 / (1.0 + np.exp(-g))) * u)).mean() > 0.05     # the sigmoid rounded instead of silu


def test_plain_model_cuts_agree_with_itself():
    # logits at position t depend on tokens 0..t only (causal), so a prefix gives the same rows
    raw = H.TINY_A
    cfg = LlamaConfig.from_dict(raw)
    t = random_tensors("LlamaForCausalLM", cfg, seed=0, dtype=torch.float32, norm_jitter=0.1)
    pm = plain.PlainLlama(raw, {k: v.numpy() for k, v in t.items()})
    toks = list(np.random.default_rng(3).integers(0, 256, size=20))
    full = pm.logits(toks)
    np.testing.assert_allclose(pm.logits(toks[:11]), full[:11], atol=1e-12)
    assert full.shape == (20, 256)
    np.testing.assert_allclose(pm.logits(toks, rows=[3, 19]), full[[3, 19]], atol=1e-12)
    # many sequences stacked (the form the tests with hundreds of requests use) give each sequence's own logits
    seqs = [toks, toks[:7], list(np.random.default_rng(4).integers(0, 256, size=33)), [5]]
    rows = [[0, 19], [6], list(range(33)), [0]]
    for r16 in (None, plain.round_bf16):
        pm.r16 = r16
        many = pm.logits_of_many(seqs, rows)
        for s, want, got in zip(seqs, rows, many):
            one = pm.logits(s, rows=want)
            assert got.shape == one.shape
            # (a product over stacked rows may add in another order: a rounding to 16 bits can fall the other way, rarely)
            close = np.abs(got - one) <= (1e-11 if r16 is None else 1e-2 * np.abs(one).max())
            assert close.all() and (np.abs(got - one) <= 1e-11).mean() > (0.999 if r16 is None else 0.9)


def test_kvmodel_writes_a_folder_that_loads(tmp_path):
    """bin/kvmodel as a program: a configuration and a seed give config.json + model.safetensors
    whose tensors are the ones the architecture declares; the same seed gives the same bytes."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    tool = os.path.join(root, "bin", "kvmodel")
    outs = []
    for k in range(2):
        d = tmp_path / f"m{k}"
        p = subprocess.run([sys.executable, tool, "--out", str(d), "--sizes", "tiny-b", "--weights-seed", "3", "--dtype", "fp32"],
                           capture_output=True, text=True, timeout=120)
        assert p.returncode == 0, p.stderr
        outs.append(open(d / "model.safetensors", "rb").read())
    assert outs[0] == outs[1]
    raw = json.load(open(tmp_path / "m0" / "config.json"))
    assert raw["architectures"] == ["LlamaForCausalLM"] and raw["num_key_value_heads"] == 1 and raw["torch_dtype"] == "float32"
    from kvcm_amd.config.model_config import LlamaConfig
    from kvcm_amd.weights.random_init import expected_tensors
    t = plain.read_safetensors(str(tmp_path / "m0" / "model.safetensors"))
    want = expected_tensors("LlamaForCausalLM", LlamaConfig.from_dict(raw))
    assert set(t) == set(want) and all(tuple(t[n].shape) == want[n][0] for n in t)
    bad = subprocess.run([sys.executable, tool, "--out", str(tmp_path / "x"), "--sizes", "nope"], capture_output=True, text=True)
    assert bad.returncode == 1 and "unknown --sizes" in bad.stderr


def test_kvcorrect_refs_container_round_trips(tmp_path):
    """The reference's KVPR file (src/main_correct.cpp:30-58): written and read back field by field;
    a wrong magic and a truncated file are refused."""
    from kvcm_amd.cli.kvcorrect import load_refs, write_refs
    rng = np.random.default_rng(3)
    steps, topk = 6, 5
    refs = [dict(prompt=rng.integers(0, 100, size=n).tolist(), greedy=rng.integers(0, 100, size=steps).tolist(),
                 top_ids=rng.integers(0, 100, size=(steps, topk)), top_logits=rng.normal(size=(steps, topk)).astype(np.float32))
            for n in (3, 11, 1)]
    path = str(tmp_path / "refs.bin")
    write_refs(path, refs, steps, topk)
    assert os.path.getsize(path) == 16 + sum(4 + 4 * len(r["prompt"]) + 4 * steps + 8 * steps * topk for r in refs)
    got, s, k = load_refs(path)
    assert (s, k, len(got)) == (steps, topk, 3)
    for a, b in zip(refs, got):
        assert a["prompt"] == b["prompt"] and a["greedy"] == b["greedy"]
        np.testing.assert_array_equal(a["top_ids"], b["top_ids"])
        np.testing.assert_array_equal(a["top_logits"], b["top_logits"])
    raw = open(path, "rb").read()
    open(path, "wb").write(b"XXXX" + raw[4:])
    with pytest.raises(ValueError, match="magic"):
        load_refs(path)
    open(path, "wb").write(raw[:-10])
    with pytest.raises(Exception):
        load_refs(path)
