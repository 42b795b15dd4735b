"""kvmodel: writes a model folder (config.json + model.safetensors) with random weights from a
configuration and a seed, for the other tools' --model and for bin/trace_run.  The reference has
no such mode: its only model files come from its exporter of trained weights
(tools/export_weights.py), which needs a network and is not rebuilt here.

  kvmodel --out DIR [--sizes NAME | --config-json FILE] [--weights-seed 0] [--dtype bf16|fp32]
          [--std 0.02] [--norm-jitter 0.0]
"""
import json
import sys

from .args import Args
from .common import NAMED_SIZES


def main(argv=None):
    try:
        a = Args(sys.argv[1:] if argv is None else argv)
        out = a.str("out", "")
        if not out:
            raise ValueError("give --out DIR")
        if a.has("config-json"):
            with open(a.str("config-json", "")) as f:
                raw = json.load(f)
        else:
            name = a.str("sizes", "tinyllama-1.1b")
            if name not in NAMED_SIZES:
                raise ValueError(f"unknown --sizes {name!r}; known: {sorted(NAMED_SIZES)}")
            raw = NAMED_SIZES[name]
        dtype = a.str("dtype", "bf16")
        if dtype not in ("bf16", "bfloat16", "fp32", "float32"):
            raise ValueError(f"--dtype {dtype!r}: bf16 or fp32")
        seed, std, jitter = a.i64("weights-seed", 0), a.f64("std", 0.02), a.f64("norm-jitter", 0.0)
        a.warn_unused()
        import torch

        from .. import architectures  # noqa: F401
        from ..registry import ARCHITECTURES
        from ..weights.random_init import write_model_dir
        arch = raw.get("architectures", ["LlamaForCausalLM"])[0]
        cfg = ARCHITECTURES.get(arch).config_class.from_dict(raw)
        path = write_model_dir(out, arch, cfg, seed, torch.bfloat16 if dtype in ("bf16", "bfloat16") else torch.float32,
                               std=std, norm_jitter=jitter)
        print(f"wrote {path}: {arch}, seed {seed}, {dtype}")
        return 0
    except Exception as e:                                       # a tool: one line, exit code 1
        print(f"kvmodel: {e}", file=sys.stderr)
        return 1
