"""What the command-line tools share: engine options from flags, and where the model comes from."""
import json

from ..config.engine_config import EngineConfig

# sizes that can be asked for by name when the weights are random
NAMED_SIZES = {
    "tinyllama-1.1b": dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
                           num_attention_heads=32, num_key_value_heads=4, head_dim=64, max_position_embeddings=2048,
                           rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "llama-2-7b": dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=32,
                       num_attention_heads=32, num_key_value_heads=32, head_dim=128, max_position_embeddings=4096,
                       rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "llama-3-8b": dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                       num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=8192,
                       rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "tiny-a": dict(vocab_size=256, hidden_size=64, intermediate_size=176, num_hidden_layers=2, num_attention_heads=4,
                   num_key_value_heads=2, head_dim=16, max_position_embeddings=128, rope_theta=10000.0,
                   rms_norm_eps=1e-5, tie_word_embeddings=False),
    "tiny-b": dict(vocab_size=384, hidden_size=96, intermediate_size=256, num_hidden_layers=3, num_attention_heads=3,
                   num_key_value_heads=1, head_dim=32, max_position_embeddings=256, rope_theta=500000.0,
                   rms_norm_eps=1e-6, tie_word_embeddings=True),
}


def engine_config_from_args(a, **overrides) -> EngineConfig:
    """Flag names and defaults of the reference's kvbench (src/main_bench.cpp:24-43), plus
    --dtype, --prefill-chunk, --eos-id, --no-graphs (no decode steps as HIP graphs), --no-programs
    (no steps replayed from recorded launch lists: every step through the model's parts) and
    --tune-products off|heuristic|all (which of the library's algorithms a many-row product runs) and
    --no-fold-norms (every RMS norm a launch of its own, rounding where the reference does)."""
    ec = EngineConfig(
        policy=a.str("policy", "paged"), block_size=a.i32("block-size", 16), max_seq_len=a.i32("max-seq-len", 2048),
        prefix_caching=a.flag("prefix"), num_blocks=a.i32("num-blocks", 0), watermark_blocks=a.i32("watermark", -1),
        pool_gb=a.f64("pool-gb", 1.0), max_num_seqs=a.i32("max-num-seqs", 256),
        max_batched_tokens=a.i32("max-batched-tokens", 4096), attn=a.str("attn", "auto"),
        dtype=a.str("dtype", "bfloat16"), prefill_chunk=a.i32("prefill-chunk", 0), eos_id=a.i32("eos-id", -1),
        use_graphs=not a.flag("no-graphs"), use_programs=not a.flag("no-programs"),
        tune_products=a.str("tune-products", "off"), fold_norms=not a.flag("no-fold-norms"))
    for k, v in overrides.items():
        setattr(ec, k, v)
    return ec.validate()


def make_engine(a, ec: EngineConfig):
    """--model DIR (config.json + safetensors; --weights is accepted as the same), or
    --random-weights with --sizes NAME | --config-json FILE and --weights-seed."""
    import torch

    from ..config.model_config import LlamaConfig
    from ..engine.engine import Engine
    from ..weights.random_init import random_tensors
    model_dir = a.str("model", a.str("weights", ""))
    if a.flag("random-weights"):
        if a.has("config-json"):
            with open(a.str("config-json", "")) as f:
                raw = json.load(f)
        else:
            name = a.str("sizes", "tinyllama-1.1b")
            if name not in NAMED_SIZES:
                raise ValueError(f"unknown --sizes {name!r}; known: {sorted(NAMED_SIZES)}")
            raw = NAMED_SIZES[name]
        arch = raw.get("architectures", ["LlamaForCausalLM"])[0]
        from .. import architectures  # noqa: F401
        from ..registry import ARCHITECTURES
        cfg = ARCHITECTURES.get(arch).config_class.from_dict(raw)
        dt = torch.bfloat16 if ec.dtype in ("bfloat16", "bf16") else torch.float32
        tensors = random_tensors(arch, cfg, a.i64("weights-seed", 0), dtype=dt, device="cuda:0")
        return Engine(config=ec, architecture=arch, model_config=cfg, tensors=tensors)
    if not model_dir:
        raise ValueError("give --model DIR (config.json + model.safetensors) or --random-weights")
    return Engine(model_dir, ec)
