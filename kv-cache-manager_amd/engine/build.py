"""From a model folder (or a configuration with tensors in memory) to a runner that can step:
config.json -> architecture (registry) -> parts -> weights by name -> cache groups and pages ->
work buffers.  Pool sizing and limits follow the reference (src/engine/engine.cpp:19-45)."""
import dataclasses
import os
import sys
from typing import Dict, Optional

import torch

from .. import architectures  # noqa: F401  (registers the known architectures)
from ..cache.manager import HostCore
from ..config.engine_config import EngineConfig
from ..config.model_config import ConfigError, read_config_json
from ..parts.base import BuildContext, KVCacheNeed
from ..parts.model import Model
from ..registry import ARCHITECTURES
from ..weights.loader import DictSource, FolderSource, load_weights
from .runner import ModelLimits, ModelRunner, kv_bytes_per_block, make_storages, plan_groups

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def torch_dtype(name):
    try:
        return _DTYPES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r} (bfloat16 | float32)") from None


def require_gpu(device="cuda:0"):
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine runs its model on an MI355X only (no CPU fallback)")
    return torch.device(device)


def read_model_config(model_dir):
    """-> (architecture entry, typed config)."""
    name, raw = read_config_json(model_dir)
    arch = ARCHITECTURES.get(name)
    return arch, arch.config_class.from_dict(raw)


def within_max_position(ec: EngineConfig, max_position: int) -> EngineConfig:
    """The model's own length limit against the engine's.  The reference carries max_pos in its
    weights header and never looks at it (src/model/weights.cpp:24-40): positions are rotated on the
    fly, so any length computes.  Here the engine's max_seq_len is cut down to the model's
    max_position (0: the architecture states none), with one line on stderr, unless the option
    ``beyond_max_position`` says that running past it is meant (replay of given traces does)."""
    if max_position <= 0 or ec.max_seq_len <= max_position or ec.beyond_max_position:
        return ec
    print(f"[kvcm] max_seq_len {ec.max_seq_len} exceeds the model's max_position_embeddings {max_position}: "
          f"sequences end at {max_position} tokens (EngineConfig.beyond_max_position=True lifts this)", file=sys.stderr, flush=True)
    return dataclasses.replace(ec, max_seq_len=max_position)


def build_runner(model_dir: Optional[str] = None, engine_config: Optional[EngineConfig] = None, *,
                 architecture: Optional[str] = None, model_config=None, tensors: Optional[Dict[str, torch.Tensor]] = None,
                 device="cuda:0"):
    """Either ``model_dir`` (config.json + safetensors) or ``architecture`` + ``model_config`` +
    ``tensors`` (checkpoint names -> tensors).  Returns (runner, core, model, model_config)."""
    ec = (engine_config or EngineConfig()).validate()
    dev = require_gpu(device)
    from .. import ops  # fails loudly when the HIP library cannot be loaded or built
    ops.lib()
    dtype = torch_dtype(ec.dtype)
    if model_dir is not None:
        arch, cfg = read_model_config(model_dir)
        source = FolderSource(model_dir)
    else:
        if architecture is None or model_config is None or tensors is None:
            raise ValueError("give a model folder, or architecture + model_config + tensors")
        arch, cfg, source = ARCHITECTURES.get(architecture), model_config, DictSource(tensors)
    spec = arch.build_spec(cfg)
    ec = within_max_position(ec, spec.max_position)
    model = Model(spec, BuildContext(dtype, dev, spec.hidden_size, ec.block_size, ops))
    try:
        weight_bytes = load_weights(model, source, dtype, dev)
    finally:
        source.close()

    num_blocks = ec.num_blocks
    if num_blocks <= 0:
        per_block = kv_bytes_per_block(model, ec.block_size, dtype)
        num_blocks = int(ec.pool_gb * float(1 << 30) / per_block) if per_block else 1
    if num_blocks <= 0:
        raise ValueError("the KV pool holds no page: raise pool_gb or num_blocks")
    groups = plan_groups(model, num_blocks, ec.max_num_seqs)
    core = HostCore(groups, policy=ec.policy, block_size=ec.block_size, max_seq_len=ec.max_seq_len,
                    prefix_caching=ec.prefix_caching, watermark_blocks=ec.watermark_blocks,
                    watermark_frac=ec.watermark_frac, max_num_seqs=ec.max_num_seqs,
                    max_batched_tokens=ec.max_batched_tokens, prefill_chunk=ec.prefill_chunk, eos_id=ec.eos_id)
    storages = make_storages(model, num_blocks, ec.block_size, ec.max_num_seqs, dtype, dev)
    limits = ModelLimits(
        max_tokens=max(ec.max_batched_tokens + ec.max_num_seqs, ec.max_seq_len),
        max_seqs=ec.max_num_seqs,
        max_logit_rows=ec.max_logit_rows if ec.max_logit_rows > 0 else max(ec.max_num_seqs, 512),
        max_blocks_per_seq=(ec.max_seq_len + ec.block_size - 1) // ec.block_size,
        max_context_len=ec.max_seq_len)
    runner = ModelRunner(model, core, storages, limits, dtype, dev, attn=ec.attn, fold_norms=ec.fold_norms,
                         tune_products=ec.tune_products)
    runner.weight_bytes = weight_bytes
    runner.num_blocks = num_blocks
    runner.engine_config = ec
    return runner, core, model, cfg
