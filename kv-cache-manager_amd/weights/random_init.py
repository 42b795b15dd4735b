"""Random weights from a configuration and a seed: as tensors in memory, or as a model folder
(config.json + model.safetensors) that loads like any checkpoint.

Every matrix and table is N(0, std); norm weights are 1, or 1 + N(0, norm_jitter) when a test
wants the multiply to matter.  Each tensor has its own generator keyed by (seed, tensor name), so
the values do not depend on the order of generation.  The reference has no random-weights mode
(its benchmark uses real weights with random token ids, src/main_bench.cpp:6-7).
"""
import hashlib
import json
import os
from typing import Dict

import torch

from .. import architectures  # noqa: F401  (registers the known architectures)
from ..parts.base import BuildContext
from ..parts.model import Model
from ..registry import ARCHITECTURES
from .safetensors_io import write_safetensors


def _generator(seed: int, name: str, device) -> torch.Generator:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(h[:8], "little") & ((1 << 63) - 1))
    return g


def expected_tensors(architecture: str, config) -> Dict[str, tuple]:
    """Checkpoint names -> (shape, role) of everything the architecture's parts declare."""
    arch = ARCHITECTURES.get(architecture)
    spec = arch.build_spec(config)
    model = Model(spec, BuildContext(torch.float32, torch.device("cpu"), spec.hidden_size, 16, None))
    out = {}
    for part in model.all_parts():
        for ps in part.param_specs():
            for name, shape in ps.sources:
                out[name] = (tuple(shape), ps.role)
    return out


def random_tensors(architecture: str, config, seed: int, dtype=torch.bfloat16, std=0.02, norm_jitter=0.0,
                   device="cpu") -> Dict[str, torch.Tensor]:
    tensors = {}
    for name, (shape, role) in expected_tensors(architecture, config).items():
        g = _generator(seed, name, device)
        if role == "vector":
            t = torch.ones(shape, dtype=torch.float32, device=device)
            if norm_jitter:
                t += norm_jitter * torch.randn(shape, generator=g, dtype=torch.float32, device=device)
        elif role == "index":
            raise NotImplementedError("random integer tables")
        else:
            t = torch.randn(shape, generator=g, dtype=torch.float32, device=device) * std
        tensors[name] = t.to(dtype)
    return tensors


def write_model_dir(path: str, architecture: str, config, seed: int, dtype=torch.bfloat16, std=0.02,
                    norm_jitter=0.0) -> str:
    """Writes config.json and model.safetensors; returns ``path``."""
    os.makedirs(path, exist_ok=True)
    raw = config.to_dict()
    raw["architectures"] = [architecture]
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=2)
    tensors = random_tensors(architecture, config, seed, dtype, std, norm_jitter)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      {"format": "pt", "weights_seed": seed, "std": std})
    return path
