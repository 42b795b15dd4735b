"""The Llama dense decoder as data: config.json keys -> a description of layers made of
registered parts.  Layer order, tensor names and the fusing of q/k/v and gate/up follow the
reference's step and exporter (src/model/llama.cpp:104-128, tools/export_weights.py:69-83)."""
from ..config.model_config import LlamaConfig
from .. import parts  # noqa: F401  (registers the built-in part kinds)
from ..parts.base import LayerSpec, ModelSpec, PartSpec
from ..registry import ARCHITECTURES, Architecture


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    H = cfg.hidden_size
    layers = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        position = PartSpec("rotary", {"theta": cfg.rope_theta, "dim": cfg.head_dim})
        layers.append(LayerSpec(
            name=f"layers.{l}", block="prenorm_residual",
            parts={
                "norm_mixer": PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, p + "input_layernorm."),
                "mixer": PartSpec("gqa_attention", {
                    "num_heads": cfg.num_attention_heads, "num_kv_heads": cfg.num_key_value_heads,
                    "head_dim": cfg.head_dim, "scale": cfg.head_dim ** -0.5, "window": 0,
                    "position": position}, p + "self_attn."),
                "norm_ffn": PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, p + "post_attention_layernorm."),
                "ffn": PartSpec("swiglu", {"intermediate_size": cfg.intermediate_size}, p + "mlp."),
            }))
    return ModelSpec(
        architecture="LlamaForCausalLM", hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}, "model.embed_tokens."),
        layers=tuple(layers), schedule=tuple(range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, "model.norm."),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "tied": cfg.tie_word_embeddings}, "lm_head."),
        max_position=cfg.max_position_embeddings)


ARCHITECTURES.register("LlamaForCausalLM", Architecture("LlamaForCausalLM", LlamaConfig, llama_spec))
