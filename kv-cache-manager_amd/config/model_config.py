"""Typed model configuration read from a model folder's config.json.

The reference has no config.json: its numbers come from the 64-byte header its exporter writes
(src/model/weights.cpp:24-40) out of the same checkpoint attributes (tools/export_weights.py:59-67).
The keys read here are those attributes; defaults are the exporter's (rope_theta 10000) and the
reference struct's (rms_eps 1e-5, src/model/weights.h:12-18).  No size lives in code.
"""
import json
import os
from dataclasses import asdict, dataclass, field
from typing import Optional


class ConfigError(ValueError):
    pass


# What the attention kernels take (csrc/hip/attention_generic.hip refuses anything else): 16-byte pieces of a
# head's row, and a head that fits a wave's registers.
MAX_HEAD_DIM = 256


def read_config_json(model_dir):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json")
    with open(path) as f:
        raw = json.load(f)
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list) or not isinstance(archs[0], str):
        raise ConfigError(f"{path}: 'architectures' must name the model class, e.g. [\"LlamaForCausalLM\"]")
    return archs[0], raw


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    architectures: tuple = field(default=("LlamaForCausalLM",))

    REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads")

    @classmethod
    def from_dict(cls, raw: dict) -> "LlamaConfig":
        problems = []
        for k in cls.REQUIRED:
            if not isinstance(raw.get(k), int) or isinstance(raw.get(k), bool) or raw[k] <= 0:
                problems.append(f"'{k}' must be a positive integer (got {raw.get(k)!r})")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        nh = raw["num_attention_heads"]
        nkv = raw.get("num_key_value_heads")
        nkv = nh if nkv is None else nkv
        hd = raw.get("head_dim")
        if hd is None:
            if raw["hidden_size"] % nh:
                problems.append(f"hidden_size {raw['hidden_size']} is not a multiple of num_attention_heads {nh} "
                                "and no head_dim is given")
            hd = raw["hidden_size"] // nh
        if not isinstance(nkv, int) or nkv <= 0 or nh % nkv:
            problems.append(f"num_attention_heads {nh} must be a multiple of num_key_value_heads {nkv!r}")
        if not isinstance(hd, int) or hd <= 0 or hd % 8 or hd > MAX_HEAD_DIM:
            problems.append(f"head_dim {hd!r} is not supported: the attention kernels take multiples of 8 up to "
                            f"{MAX_HEAD_DIM} (hidden_size {raw['hidden_size']}, num_attention_heads {nh})")
        scaling = raw.get("rope_scaling")
        plain_rotary = scaling in (None, {}) or (isinstance(scaling, dict) and set(scaling) <= {"rope_type", "type"}
                                                 and all(v == "default" for v in scaling.values()))
        if not plain_rotary:
            problems.append(f"rope_scaling {scaling!r} is not supported (only plain rotary positions)")
        for k in ("attention_bias", "mlp_bias"):
            if raw.get(k):
                problems.append(f"{k}=true is not supported (projections have no bias)")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            problems.append(f"hidden_act {act!r} is not supported (silu)")
        theta = raw.get("rope_theta", 10000.0)
        eps = raw.get("rms_norm_eps", 1e-5)
        if not isinstance(theta, (int, float)) or theta <= 0:
            problems.append(f"rope_theta {theta!r} must be positive")
        if not isinstance(eps, (int, float)) or eps <= 0:
            problems.append(f"rms_norm_eps {eps!r} must be positive")
        max_pos = raw.get("max_position_embeddings", 2048)
        if not isinstance(max_pos, int) or max_pos <= 0:
            problems.append(f"max_position_embeddings {max_pos!r} must be a positive integer")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cls(vocab_size=raw["vocab_size"], hidden_size=raw["hidden_size"],
                   intermediate_size=raw["intermediate_size"], num_hidden_layers=raw["num_hidden_layers"],
                   num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd,
                   max_position_embeddings=max_pos, rope_theta=float(theta), rms_norm_eps=float(eps),
                   tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)), hidden_act=act,
                   torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
                   architectures=tuple(raw.get("architectures", ("LlamaForCausalLM",))))

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        return d

    # derived sizes (src/model/weights.h:16-17)
    @property
    def q_dim(self): return self.num_attention_heads * self.head_dim
    @property
    def kv_dim(self): return self.num_key_value_heads * self.head_dim
    @property
    def qkv_dim(self): return self.q_dim + 2 * self.kv_dim

    def num_parameters(self) -> int:
        H, I, V = self.hidden_size, self.intermediate_size, self.vocab_size
        per_layer = 2 * H + self.qkv_dim * H + H * self.q_dim + 3 * I * H
        return V * H + self.num_hidden_layers * per_layer + H + (0 if self.tie_word_embeddings else V * H)
