"""Weights by tensor name.

Every part of a model declares the tensors it wants (ParamSpec: checkpoint names, shapes, how to
fuse them).  The loader checks the whole checkpoint against the whole model first and reports,
in one error, every missing tensor, every unexpected one and every wrong shape; only then does it
move data.  The reference fuses q/k/v and gate/up in its exporter (tools/export_weights.py:69-83)
and has no by-name loading; the fusing here happens at load time on the device.

Stored precision: matrices and tables take the compute dtype (bfloat16 when serving, float32 in
the 32-bit path); a vector that the checkpoint stores in 32 bits stays 32-bit; integer tables
become int32.
"""
import json
import os
from typing import Dict, Iterable

import torch

from .safetensors_io import SafetensorsFile


class WeightsError(ValueError):
    pass


class DictSource:
    """Tensors already in memory (random weights, tests)."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self.tensors = tensors

    def names(self): return list(self.tensors)
    def shape(self, name): return tuple(self.tensors[name].shape)
    def dtype(self, name): return self.tensors[name].dtype
    def get(self, name): return self.tensors[name]
    def close(self): pass


class FolderSource:
    """model.safetensors, or the shards that model.safetensors.index.json names."""

    def __init__(self, model_dir):
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        files = []
        if os.path.isfile(single):
            files = [single]
        elif os.path.isfile(index):
            with open(index) as f:
                files = sorted({os.path.join(model_dir, v) for v in json.load(f)["weight_map"].values()})
        else:
            files = sorted(os.path.join(model_dir, f) for f in os.listdir(model_dir) if f.endswith(".safetensors"))
        if not files:
            raise WeightsError(f"{model_dir}: no model.safetensors (nor shards) found")
        self.files = [SafetensorsFile(p) for p in files]
        self.where = {}
        for sf in self.files:
            for n in sf.names():
                if n in self.where:
                    raise WeightsError(f"tensor {n} is stored in two files")
                self.where[n] = sf

    def names(self): return list(self.where)
    def shape(self, name): return self.where[name].shape(name)
    def dtype(self, name): return self.where[name].dtype(name)
    def get(self, name): return self.where[name].tensor(name)

    def close(self):
        for sf in self.files:
            sf.close()


def _stored_dtype(role, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if role == "index":
        if stored.is_floating_point:
            raise WeightsError("an integer table is stored as floating point")
        return torch.int32
    if not stored.is_floating_point:
        raise WeightsError("a floating-point tensor is stored as integers")
    if compute == torch.float32:
        return torch.float32
    if role == "vector" and stored in (torch.float32, torch.float64):
        return torch.float32
    return compute


def check_against(model, source) -> None:
    """Raises one WeightsError listing every missing, unexpected and misshapen tensor."""
    expected, ignorable = {}, set()
    for part in model.all_parts():
        for spec in part.param_specs():
            for name, shape in spec.sources:
                expected[name] = tuple(shape)
        ignorable.update(part.ignorable_tensors())
    have = set(source.names())
    missing = sorted(n for n in expected if n not in have)
    unexpected = sorted(n for n in have if n not in expected and n not in ignorable)
    wrong = sorted((n, expected[n], source.shape(n)) for n in expected if n in have and source.shape(n) != expected[n])
    if not (missing or unexpected or wrong):
        return
    lines = ["the checkpoint does not fit the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}): " +
                     ", ".join(f"{n} expected {list(e)} got {list(g)}" for n, e, g in wrong))
    raise WeightsError("\n".join(lines))


def load_weights(model, source, compute_dtype: torch.dtype, device) -> int:
    """Checks, then binds every part's tensors on ``device``.  Returns the bytes now on the device."""
    check_against(model, source)
    total = 0
    for part in model.all_parts():
        bound = {}
        for spec in part.param_specs():
            dtypes = {_stored_dtype(spec.role, source.dtype(n), compute_dtype) for n, _ in spec.sources}
            if len(dtypes) != 1:
                raise WeightsError(f"{spec.sources[0][0]} and the tensors fused with it are stored in different precisions")
            dt = dtypes.pop()
            out = torch.empty(spec.shape, dtype=dt, device=device)
            row = 0
            for name, shape in spec.sources:
                out[row:row + shape[0]].copy_(source.get(name).to(dt))
                row += shape[0]
            bound[spec.name] = out
            total += out.numel() * out.element_size()
        part.bind(bound)
    model.finish_binding()
    return total
