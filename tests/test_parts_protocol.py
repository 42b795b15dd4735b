"""What parts declare about themselves and what the engine does with it (no GPU): which registry a
named part of a block arrangement comes from, when a model's steps may be recorded and replayed,
the garbage-collection guard around a capture, and the model's own length limit."""
import gc

import pytest
import torch

import helpers as H
from kvcm_amd import architectures  # noqa: F401
from kvcm_amd.config.engine_config import EngineConfig
from kvcm_amd.config.model_config import LlamaConfig
from kvcm_amd.engine.build import within_max_position
from kvcm_amd.parts.base import Block, BuildContext, FeedForward, KVCacheNeed, LayerSpec, Mixer, ModelSpec, PartSpec, StateNeed
from kvcm_amd.parts.model import Model, _registry_for
from kvcm_amd.registry import ARCHITECTURES, BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Registry


def _ctx(width):
    return BuildContext(torch.float32, torch.device("cpu"), width, 16, None)


def _llama(raw):
    spec = ARCHITECTURES.get("LlamaForCausalLM").build_spec(LlamaConfig.from_dict(raw))
    return Model(spec, _ctx(spec.hidden_size))


# ---------------------------------------------------------------- registries of a block's parts
def test_common_part_names_need_no_declaration():
    assert _registry_for("mixer") is MIXERS and _registry_for("ffn") is FEED_FORWARDS
    assert _registry_for("norm_mixer") is NORMS and _registry_for("norm") is NORMS
    with pytest.raises(KeyError, match="part_registries"):
        _registry_for("router")


def test_a_block_arrangement_names_the_registries_of_its_own_parts():
    gates = Registry("gate")

    class Gated(Block):
        part_registries = {"router": "feed_forward", "second_mixer": "mixer", "gate": gates, "place": "position",
                           "mixer": gates}      # may also re-route a common name

    assert _registry_for("router", Gated) is FEED_FORWARDS
    assert _registry_for("second_mixer", Gated) is MIXERS
    assert _registry_for("gate", Gated) is gates and _registry_for("mixer", Gated) is gates
    assert _registry_for("place", Gated) is POSITIONS
    assert _registry_for("norm_in", Gated) is NORMS            # undeclared names keep their common meaning
    with pytest.raises(KeyError, match="part_registries"):
        _registry_for("extra", Gated)

    class Wrong(Block):
        part_registries = {"router": "routers"}

    with pytest.raises(KeyError, match="names no registry"):
        _registry_for("router", Wrong)


def test_a_model_is_built_with_a_block_that_has_two_mixers_and_a_router():
    """The layer's part names go through the arrangement's declaration: nothing in the package
    knows the names "left", "right" or "router"."""
    built = []

    class Probe(Mixer):
        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            built.append(("mixer", prefix))

    class Route(FeedForward):
        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            built.append(("route", prefix))

    class TwoMixers(Block):
        part_registries = {"left": "mixer", "right": "mixer", "router": "feed_forward"}

    MIXERS.register("probe_mixer_for_protocol_test", Probe)
    FEED_FORWARDS.register("probe_route_for_protocol_test", Route)
    BLOCKS.register("probe_two_mixers", TwoMixers)
    layer = LayerSpec("only", "probe_two_mixers", {
        "left": PartSpec("probe_mixer_for_protocol_test", {}, "l."), "right": PartSpec("probe_mixer_for_protocol_test", {}, "r."),
        "router": PartSpec("probe_route_for_protocol_test", {}, "g."), "norm_in": PartSpec("rmsnorm", {"size": 8, "eps": 1e-5}, "n.")})
    spec = ModelSpec("Probe", 8, 11, PartSpec("token_embedding", {"vocab_size": 11}, "e."), (layer,), (0,),
                     PartSpec("rmsnorm", {"size": 8, "eps": 1e-5}, "f."), PartSpec("linear_head", {"vocab_size": 11, "tied": True}, "h."))
    model = Model(spec, _ctx(8))
    assert sorted(built) == [("mixer", "l."), ("mixer", "r."), ("route", "g.")]
    assert isinstance(model.blocks[0], TwoMixers) and set(model.layer_parts[0]) == {"left", "right", "router", "norm_in"}
    assert not model.capturable and "TwoMixers" in model.not_capturable() and "Probe" in model.not_capturable()


# ------------------------------------------------------------------------------ recording steps
def test_llama_is_capturable_and_says_so_part_by_part():
    model = _llama(H.TINY_A)
    kinds = {type(p).__name__ for p in model.every_part()}
    assert {"RMSNorm", "GQAAttention", "Rotary", "SwiGLU", "TokenEmbedding", "LinearHead"} <= kinds     # the rotary is a sub-part
    assert all(p.capturable for p in model.every_part()) and all(b.capturable for b in model.blocks)
    assert model.capturable and model.not_capturable() == []


def test_one_part_that_reads_host_values_keeps_the_whole_model_off_recorded_steps():
    class Stateful(Mixer):          # says nothing about itself: the default must be the safe one
        def cache_need(self):
            return StateNeed((4,), torch.float32)

    MIXERS.register("stateful_for_protocol_test", Stateful)
    raw = dict(H.TINY_A)
    spec = ARCHITECTURES.get("LlamaForCausalLM").build_spec(LlamaConfig.from_dict(raw))
    first = spec.layers[0]
    parts = dict(first.parts)
    parts["mixer"] = PartSpec("stateful_for_protocol_test", {}, "x.")
    layers = (LayerSpec(first.name, first.block, parts),) + tuple(spec.layers[1:])
    model = Model(ModelSpec(spec.architecture, spec.hidden_size, spec.vocab_size, spec.embedding, layers, spec.schedule,
                            spec.final_norm, spec.head), _ctx(spec.hidden_size))
    assert Stateful.capturable is False
    assert not model.capturable and model.not_capturable() == ["Stateful"]


def test_no_garbage_collection_during_a_capture_and_the_old_state_comes_back():
    from kvcm_amd.engine.graphs import _no_collection
    assert gc.isenabled()
    with _no_collection():
        assert not gc.isenabled()
        with _no_collection():              # nested: still off inside, still off after the inner one
            assert not gc.isenabled()
        assert not gc.isenabled()
    assert gc.isenabled()
    with pytest.raises(RuntimeError):
        with _no_collection():
            raise RuntimeError("capture failed")
    assert gc.isenabled()
    gc.disable()
    try:
        with _no_collection():
            assert not gc.isenabled()
        assert not gc.isenabled()           # it was off before: it stays off
    finally:
        gc.enable()


# ------------------------------------------------------------------- the model's own length limit
def test_max_seq_len_is_cut_down_to_the_models_max_position(capsys):
    ec = EngineConfig(max_seq_len=2048)
    cut = within_max_position(ec, 128)
    assert cut.max_seq_len == 128 and ec.max_seq_len == 2048
    assert "max_position_embeddings 128" in capsys.readouterr().err
    assert within_max_position(EngineConfig(max_seq_len=64), 128).max_seq_len == 64
    assert within_max_position(EngineConfig(max_seq_len=2048), 0).max_seq_len == 2048           # the architecture states none
    assert within_max_position(EngineConfig(max_seq_len=2048, beyond_max_position=True), 128).max_seq_len == 2048
    assert capsys.readouterr().err == ""


# ------------------------------------------------------------- refusals where the model is built
def test_attention_refuses_a_head_size_its_kernels_do_not_take_when_it_is_built():
    """Not at the first step's launch: a configuration that reaches the part some other way than
    through LlamaConfig (another architecture's description) is refused with the sizes named."""
    from kvcm_amd.parts.llama_parts import GQAAttention
    position = PartSpec("none", {})
    for hd in (12, 20, 264):
        with pytest.raises(ValueError, match=f"head_dim {hd} is not supported"):
            GQAAttention({"num_heads": 4, "num_kv_heads": 2, "head_dim": hd, "position": position}, "a.", _ctx(64))
    with pytest.raises(ValueError, match="not a multiple of num_kv_heads"):
        GQAAttention({"num_heads": 4, "num_kv_heads": 3, "head_dim": 16, "position": position}, "a.", _ctx(64))
    GQAAttention({"num_heads": 4, "num_kv_heads": 2, "head_dim": 8, "position": position}, "a.", _ctx(64))
    GQAAttention({"num_heads": 4, "num_kv_heads": 2, "head_dim": 256, "position": position}, "a.", _ctx(64))


# --------------------------------------------------------------- several cache owners in a layer
def test_every_part_of_a_layer_that_needs_a_cache_gets_one_under_any_name():
    """An attention beside a state mixer in one layer, under names the package does not know; a
    second layer whose parts read the first layer's caches, one by a layer name, one by layer.part."""
    class Keys(Mixer):
        def cache_need(self):
            return KVCacheNeed(2, 16, 0)

    class State(Mixer):
        def cache_need(self):
            return StateNeed((4,), torch.float32)

    class Gate(FeedForward):            # not a mixer, and it keeps something per request all the same
        def cache_need(self):
            return StateNeed((2,), torch.float32)

    class Pair(Block):
        part_registries = {"look": "mixer", "remember": "mixer", "gate": "feed_forward"}

    MIXERS.register("keys_for_owner_test", Keys)
    MIXERS.register("state_for_owner_test", State)
    FEED_FORWARDS.register("gate_for_owner_test", Gate)
    BLOCKS.register("pair_for_owner_test", Pair)

    def layer(name, cache_from=None):
        return LayerSpec(name, "pair_for_owner_test", {
            "look": PartSpec("keys_for_owner_test", {}, name + ".k."), "remember": PartSpec("state_for_owner_test", {}, name + ".s."),
            "gate": PartSpec("gate_for_owner_test", {}, name + ".g.")}, cache_from)

    def model(layers):
        spec = ModelSpec("Probe", 8, 11, PartSpec("token_embedding", {"vocab_size": 11}, "e."), tuple(layers), tuple(range(len(layers))),
                         PartSpec("rmsnorm", {"size": 8, "eps": 1e-5}, "f."), PartSpec("linear_head", {"vocab_size": 11, "tied": True}, "h."))
        return Model(spec, _ctx(8))

    m = model([layer("a"), layer("b"), layer("c", {"look": "a", "remember": "b.remember"})])
    assert [(type(g.need).__name__, g.layers) for g in m.groups] == [
        ("KVCacheNeed", [("a", "look"), ("b", "look")]),
        ("StateNeed", [("a", "remember"), ("b", "remember")]),
        ("StateNeed", [("a", "gate"), ("b", "gate"), ("c", "gate")])]          # c's gate is not listed: it keeps its own

    class Store:
        def __init__(self, g):
            self.group = g

    m.attach_caches([Store(0), Store(1), Store(2)])
    got = {(l.name, slot): (p.cache.group, p.cache_index, p.cache_owner)
           for l, parts in zip(m.spec.layers, m.layer_parts) for slot, p in parts.items()}
    assert got == {("a", "look"): (0, 0, True), ("a", "remember"): (1, 0, True), ("a", "gate"): (2, 0, True),
                   ("b", "look"): (0, 1, True), ("b", "remember"): (1, 1, True), ("b", "gate"): (2, 1, True),
                   ("c", "look"): (0, 0, False), ("c", "remember"): (1, 1, False), ("c", "gate"): (2, 2, True)}
    # one string for the whole layer: every cache-using part reads the part of its own name there
    whole = model([layer("a"), layer("r", "a")])
    assert [g.layers for g in whole.groups] == [[("a", "look")], [("a", "remember")], [("a", "gate")]]
    with pytest.raises(ValueError, match="names no layer"):
        model([layer("a"), layer("r", "nowhere")])
    with pytest.raises(ValueError, match="which owns none"):
        model([layer("a"), layer("r", {"look": "a.remember2"})])
    with pytest.raises(ValueError, match="does not have"):
        model([layer("a"), layer("r", {"lok": "a"})])


def test_norms_fold_up_to_fewer_rows_the_wider_the_layers():
    """Rows x a layer's weight bytes up to a constant fold: 8 rows at TinyLlama sizes, 2 at 7B / 8B sizes, never
    fewer than one."""
    from kvcm_amd.engine.runner import ModelRunner
    tiny = 2 * (2560 * 2048 + 2048 * 2048 + 2 * 5632 * 2048 + 2048 * 5632)           # bfloat16 bytes of a layer
    eight_b = 2 * (6144 * 4096 + 4096 * 4096 + 2 * 14336 * 4096 + 4096 * 14336)
    seven_b = 2 * (3 * 4096 * 4096 + 4096 * 4096 + 3 * 11008 * 4096)
    assert ModelRunner.fold_rows_for(tiny, 8) == 8 and ModelRunner.fold_rows_for(eight_b, 8) == 2
    assert ModelRunner.fold_rows_for(seven_b, 8) == 2 and ModelRunner.fold_rows_for(5e9, 8) == 1
    assert ModelRunner.fold_rows_for(1e6, 8) == 8 and ModelRunner.fold_rows_for(tiny, 4) == 4
