"""Random weights from a configuration and a seed: as tensors in memory, or as a model folder
(config.json + model.safetensors) that loads like any checkpoint.

Every matrix and table is N(0, std); norm weights are 1, or 1 + N(0, norm_jitter) when a test
wants the multiply to matter.  The values come from a counter-based rule keyed by (seed, tensor
name, element index): they depend neither on the order in which tensors are made nor on where they
are made.  On the host NumPy evaluates the rule, on the GPU the ``fill_normal`` kernel
(csrc/hip/fill_normal.hip); both give the same numbers (the last bit of a 32-bit value may differ
for about one element in 10^8, where the two math libraries round a logarithm or cosine differently).
The reference has no random-weights mode (its benchmark uses real weights with random token ids,
src/main_bench.cpp:6-7).

The rule:  mix = SplitMix64's output function;  key = mix(mix(seed) ^ fnv1a64(name));
z1 = mix(key + (i + 1) * 0x9E3779B97F4A7C15), z2 = mix(z1);  u1 = ((z1 >> 12) + 0.5) / 2^52,
u2 = (z2 >> 12) / 2^52;  n_i = sqrt(-2 ln u1) cos(2 pi u2) in double precision, cast to float32;
value = float32(mean + std * n_i), then the storage type.
"""
import json
import os
from typing import Dict

import numpy as np
import torch

from .. import architectures  # noqa: F401  (registers the known architectures)
from ..parts.base import BuildContext
from ..parts.model import Model
from ..registry import ARCHITECTURES
from .safetensors_io import write_safetensors

_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
INDEX_MODULUS = 1024          # random integer tables hold values in [0, INDEX_MODULUS)


def _mix_int(z: int) -> int:
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def tensor_key(seed: int, name: str) -> int:
    h = 0xCBF29CE484222325
    for byte in name.encode():
        h = ((h ^ byte) * 0x100000001B3) & _M64
    return _mix_int(_mix_int(seed & _M64) ^ h)


def _counters(key: int, start: int, count: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        return _mix(np.uint64(key) + i * np.uint64(_GOLDEN))


def normal_values(key: int, count: int, chunk: int = 1 << 22) -> np.ndarray:
    """The rule's standard normal values n_0 .. n_{count-1} as float32, evaluated on the host."""
    out = np.empty(count, dtype=np.float32)
    for lo in range(0, count, chunk):
        n = min(chunk, count - lo)
        with np.errstate(over="ignore"):
            z1 = _counters(key, lo, n)
            z2 = _mix(z1)
        u1 = ((z1 >> np.uint64(12)).astype(np.float64) + 0.5) * (1.0 / 4503599627370496.0)
        u2 = (z2 >> np.uint64(12)).astype(np.float64) * (1.0 / 4503599627370496.0)
        out[lo:lo + n] = (np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925286766559 * u2)).astype(np.float32)
    return out


def index_values(key: int, count: int, modulus: int = INDEX_MODULUS) -> np.ndarray:
    return (_counters(key, 0, count) % np.uint64(modulus)).astype(np.int32)


def random_tensor(seed: int, name: str, shape, role: str, dtype=torch.bfloat16, std=0.02, norm_jitter=0.0, device="cpu"):
    """One tensor of the rule.  role "vector": 1 + norm_jitter * n; "index": int32 in [0, INDEX_MODULUS);
    else std * n.  On a GPU the fill kernel makes the values in place."""
    key = tensor_key(seed, name)
    dev = torch.device(device)
    count = int(np.prod(shape)) if len(shape) else 1
    mean, scale = (1.0, float(norm_jitter)) if role == "vector" else (0.0, float(std))
    if dev.type == "cuda":
        from .. import ops
        if role == "index":
            return ops.fill_index(torch.empty(shape, dtype=torch.int32, device=dev), key, INDEX_MODULUS)
        store = dtype if dtype in (torch.float32, torch.bfloat16) else torch.float32
        t = torch.empty(shape, dtype=store, device=dev)
        if scale == 0.0:
            t.fill_(mean)
        else:
            ops.fill_normal(t, key, mean, scale)
        return t.to(dtype)
    if role == "index":
        return torch.from_numpy(index_values(key, count).reshape(shape))
    if scale == 0.0:
        return torch.full(shape, mean, dtype=torch.float32).to(dtype)
    values = np.float32(mean) + np.float32(scale) * normal_values(key, count)          # float32 arithmetic, as on the device
    return torch.from_numpy(values.reshape(shape)).to(dtype)


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
    return {name: random_tensor(seed, name, shape, role, dtype, std, norm_jitter, device)
            for name, (shape, role) in expected_tensors(architecture, config).items()}


def write_model_dir(path: str, architecture: str, config, seed: int, dtype=torch.bfloat16, std=0.02,
                    norm_jitter=0.0, device=None) -> str:
    """Writes config.json and model.safetensors; returns ``path``.  The values are made on ``device``
    (default: the GPU when one is visible, which takes seconds where the host takes minutes at served
    sizes; the numbers are the same either way)."""
    if device is None:
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    os.makedirs(path, exist_ok=True)
    raw = config.to_dict()
    raw["architectures"] = [architecture]
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=2)
    tensors = {k: v.cpu() for k, v in random_tensors(architecture, config, seed, dtype, std, norm_jitter, device).items()}
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      {"format": "pt", "weights_seed": seed, "std": std})
    return path
