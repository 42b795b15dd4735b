"""A small, whole inference engine for one GPU (AMD MI355X, gfx950): from a model folder to
the next token.  Sub-packages: config, weights, parts, architectures, cache, engine, sampling,
csrc (native host core and HIP kernels), cli.

    from kvcm_amd import Engine, EngineConfig
    eng = Engine("path/to/model", EngineConfig(dtype="bfloat16"))
    outputs = eng.generate([[1, 2, 3], [4, 5]], max_new_tokens=16)
"""
__version__ = "0.1.0"

_LAZY = {
    "Engine": ("engine.engine", "Engine"),
    "StepInfo": ("engine.engine", "StepInfo"),
    "EngineConfig": ("config.engine_config", "EngineConfig"),
    "LlamaConfig": ("config.model_config", "LlamaConfig"),
    "TraceReplayer": ("engine.replay", "TraceReplayer"),
    "write_model_dir": ("weights.random_init", "write_model_dir"),
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        mod, attr = _LAZY[name]
        return getattr(importlib.import_module(f"{__name__}.{mod}"), attr)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def generate(model_dir, prompts, max_new_tokens, temperature=0.0, seed=0, **engine_options):
    """One call from a model folder to generated token ids (a list per prompt)."""
    from .config.engine_config import EngineConfig
    from .engine.engine import Engine
    return Engine(model_dir, EngineConfig(**engine_options)).generate(prompts, max_new_tokens, temperature, seed)
