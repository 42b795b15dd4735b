"""Engine options.  Names, meanings and defaults are the reference's where it has them
(EngineConfig src/engine/engine.h:16-22, KVManagerConfig src/core/kv_manager.h:64-72,
SchedulerConfig src/core/scheduler.h:14-18); dtype, prefill_chunk, eos_id and the sampler
fields are additions."""
from dataclasses import dataclass


@dataclass
class EngineConfig:
    policy: str = "paged"            # "paged" | "contiguous"
    block_size: int = 16
    max_seq_len: int = 2048
    prefix_caching: bool = False
    num_blocks: int = 0              # <= 0: derived from pool_gb
    pool_gb: float = 1.0
    watermark_blocks: int = -1       # -1: watermark_frac of the pool
    watermark_frac: float = 0.01
    max_num_seqs: int = 256
    max_batched_tokens: int = 4096
    prefill_chunk: int = 0           # 0: prompts are scheduled whole, as in the reference
    eos_id: int = -1                 # -1: the end-of-sequence token is ignored, as in the reference
    attn: str = "auto"               # "v1" | "v2" | "auto"
    max_logit_rows: int = 0          # 0: max(max_num_seqs, 512)
    dtype: str = "bfloat16"          # "bfloat16" | "float32"
    use_graphs: bool = True          # replay decode-only steps from captured HIP graphs (models whose parts are all capturable)
    use_programs: bool = True        # replay other step shapes from natively recorded launch lists (same condition)
    beyond_max_position: bool = False  # False: max_seq_len is cut down to the model's max_position_embeddings (with a notice)
    fold_norms: bool = True            # bfloat16 decode steps of a few rows (up to 8; fewer for wide models, where it stops
                                       # paying earlier) fold their RMS norms into the products around them (two roundings at
                                       # other places than the reference's, same size); False: every norm is a launch of its
                                       # own and rounds exactly where the reference does
    tune_products: str = "off"         # which library algorithm a many-row product runs: "off" the library's first choice,
                                       # "heuristic" its choices timed at a shape's first use (tens of milliseconds per shape,
                                       # about 5 % of the product's time afterwards), "all" every algorithm (seconds per shape)

    def validate(self):
        if self.policy not in ("paged", "contiguous"):
            raise ValueError(f"unknown KV policy: {self.policy} (paged | contiguous)")
        if self.attn not in ("v1", "v2", "auto"):
            raise ValueError(f"unknown attention version: {self.attn} (v1 | v2 | auto)")
        if self.dtype not in ("bfloat16", "float32", "bf16", "fp32"):
            raise ValueError(f"unknown dtype: {self.dtype} (bfloat16 | float32)")
        if self.tune_products not in ("off", "heuristic", "all"):
            raise ValueError(f"unknown tune_products: {self.tune_products} (off | heuristic | all)")
        for name in ("block_size", "max_seq_len", "max_num_seqs", "max_batched_tokens"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive")
        return self
