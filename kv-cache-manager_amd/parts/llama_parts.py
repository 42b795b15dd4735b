"""The parts a Llama-style decoder is made of: RMS norm, rotary positions, grouped-query attention
over the paged cache, SwiGLU feed-forward, token embedding, output head, and the pre-norm residual
arrangement.  Formulas and rounding points follow the reference step (src/model/llama.cpp:84-128)
and its kernels (src/cuda/kernels.cu, src/cuda/paged_attention.cu); every size and constant is a
parameter.
"""
import math

import torch

from ..registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS
from . import paged_attention
from .base import (Block, Embedding, FeedForward, Head, KVCacheNeed, Mixer, Norm, ParamSpec, PositionEncoding, as_tensor)


def _linear(ctx, step, x, w, name, keep_partial=False, dtype=None):
    """x @ w^T into the work buffer ``name``.  With ``keep_partial`` the result may come back as
    un-added split-K sums (ops.PartialSums) for a consumer that adds them up itself."""
    out = step.ws(name, (x.shape[0], w.shape[0]), dtype)
    scratch = step.scratch(name, x.shape[0], w.shape[0], w.shape[1])
    return ctx.ops.gemm(x, w, out, scratch=scratch, keep_partial=keep_partial and scratch is not None,
                        tuning=step.tune_products)


def _to_residual(ctx, step, x, w, name):
    """A part's last product, whose result goes to the residual stream.  For decode steps of a few
    rows it is handed on unrun (ops.PendingProduct): the norm that follows runs it with the addition
    and its own preparation in the epilogue.  Otherwise it runs here, split sums left un-added."""
    ops = ctx.ops
    if (step.fold_norms and x.dtype == torch.bfloat16 and x.shape[0] <= min(ops.FUSED_NORM_MAX_ROWS, step.fold_rows)
            and ops.gemm8_supported(x.shape[0], w.shape[0], w.shape[1])):
        out = step.ws(name, (x.shape[0], w.shape[0]))
        return ops.PendingProduct(x, w, out, step.scratch(name, x.shape[0], w.shape[0], w.shape[1]))
    return _linear(ctx, step, x, w, name, keep_partial=True)


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """out = weight * round(x / sqrt(mean(x^2) + eps)); eps inside the root, no mean removed, the
    weight a plain multiplier (src/cuda/kernels.cu:34-49).  params: size, eps."""

    capturable = True
    accepts_partial_sums = True
    defers = True

    def param_specs(self):
        return [ParamSpec("weight", ((self.prefix + "weight", (self.params["size"],)),), role="vector")]

    def bind(self, tensors):
        super().bind(tensors)
        # where the folded form of this norm leaves its rows (ops.NormedRows), kept for good: recorded
        # steps hold the addresses
        H, ops = self.params["size"], self.ctx.ops
        self._folded = None
        if ops is not None and self.ctx.dtype == torch.bfloat16 and H % 8 == 0 and self.ctx.device.type == "cuda":
            self._folded = (torch.empty(ops.FUSED_NORM_MAX_ROWS, H, dtype=torch.bfloat16, device=self.ctx.device),
                            torch.empty(ops.FUSED_NORM_MAX_ROWS, H // 8, dtype=torch.float32, device=self.ctx.device))

    def forward(self, x, out, add=None, rows=None, defer=False):
        ops = self.ctx.ops
        if isinstance(add, ops.PendingProduct):
            if (defer and rows is None and self._folded is not None and add.x.shape[0] == x.shape[0] <= ops.FUSED_NORM_MAX_ROWS
                    and add.dtype == torch.bfloat16):
                return ops.gemm_residual_norm(add, x, self.w["weight"], self.params["eps"], *self._folded, out)
            add = add.run(keep_partial=True)
        ops.rmsnorm(x, self.w["weight"], out, self.params["eps"], add=add, rows=rows)
        return out


@POSITIONS.register("rotary")
class Rotary(PositionEncoding):
    """Rotate-half rotary positions over the first ``dim`` (= head_dim) entries of every q and k
    head: pairs (j, j + dim/2), inv_freq_j = theta^(-2j/dim), angle = position * inv_freq_j in
    32-bit (src/cuda/kernels.cu:51-70).  params: theta, dim."""

    capturable = True
    accepts_partial_sums = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        dim = params["dim"]
        j = torch.arange(0, dim, 2, dtype=torch.float32)
        self.inv_freq = (1.0 / torch.pow(torch.tensor(float(params["theta"]), dtype=torch.float32), j / dim)).to(ctx.device)

    def ignorable_tensors(self):
        return (self.prefix + "rotary_emb.inv_freq",)

    def rotation_table(self, step, head_dim):
        """(cos, sin) of every row's angles [rows, head_dim/2, 2].  The angles depend on the row
        only: the first layer of a step computes them, the others with the same theta and dim read
        them.  Each (theta, dim) has a table and a work buffer of its own, so layers that alternate
        between two thetas do not overwrite each other's angles."""
        if head_dim != self.params["dim"]:
            return None
        theta = float(self.params["theta"])
        key = ("rotary", theta, head_dim)
        table = step.shared.get(key)
        if table is None:
            name = "rotary_cos_sin_%d_%s" % (head_dim, theta.hex())
            table = step.ws(name, (step.rows, head_dim), torch.float32).view(step.rows, head_dim // 2, 2)
            self.ctx.ops.rope_table(step.positions, self.inv_freq, table, rows=step.rows)
            step.shared[key] = table
        return table

    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None, source=None):
        if head_dim != self.params["dim"]:
            raise ValueError("rotary: this kernel rotates the whole head (dim must equal head_dim)")
        k, v = cache if cache is not None else (None, None)
        table = self.rotation_table(step, head_dim)
        self.ctx.ops.rope_cache(qkv, num_heads, num_kv_heads, head_dim, positions=step.positions,
                                inv_freq=self.inv_freq, slots=slots, kcache=k, vcache=v,
                                block_size=self.ctx.block_size, rows=step.rows, source=source, cos_sin=table)
        return cache is not None


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    capturable = True
    rotates = False

    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
        return False


@MIXERS.register("gqa_attention")
class GQAAttention(Mixer):
    """Grouped-query attention over the paged cache.  One fused projection [q | k | v]
    (src/model/llama.cpp:108), positions applied to q and k, k and v stored to the pages of this
    step's rows before attention reads them (llama.cpp:111-115), so a portion of a prompt attends
    to itself through the cache; causality is context length = position + 1.
    params: num_heads, num_kv_heads, head_dim, scale, window (0 = all keys), position (PartSpec)."""

    capturable = True
    accepts_normed_rows = True

    def sub_parts(self):
        return (self.position,)

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.nkv, self.hd = p["num_heads"], p["num_kv_heads"], p["head_dim"]
        # refused where the model is built, not at the first step's launch
        if self.hd <= 0 or self.hd % 8 or self.hd > 256:
            raise ValueError(f"gqa_attention {prefix!r}: head_dim {self.hd} is not supported (the attention kernels take "
                             f"multiples of 8 up to 256; num_heads {self.nh}, num_kv_heads {self.nkv})")
        if self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"gqa_attention {prefix!r}: num_heads {self.nh} is not a multiple of num_kv_heads {self.nkv}")
        self.scale = p.get("scale", 1.0 / math.sqrt(self.hd))
        self.window = p.get("window", 0)
        pos = p["position"]
        self.position = POSITIONS.get(pos.kind)(pos.params, prefix, ctx)
        self.q_dim, self.kv_dim = self.nh * self.hd, self.nkv * self.hd

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        return [ParamSpec("wqkv", ((pre + "q_proj.weight", (self.q_dim, H)), (pre + "k_proj.weight", (self.kv_dim, H)),
                                   (pre + "v_proj.weight", (self.kv_dim, H)))),
                ParamSpec("wo", ((pre + "o_proj.weight", (H, self.q_dim)),))]

    def ignorable_tensors(self):
        return self.position.ignorable_tensors()

    def cache_need(self):
        return KVCacheNeed(self.nkv, self.hd, self.window)

    def flops(self, rows, attended=0):
        # the two projections, and q.k and p.v over every (row, key) pair of every query head
        return super().flops(rows) + 4.0 * attended * self.hd * self.nh

    def forward(self, step, h):
        ops = self.ctx.ops
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        pos = self.position
        res = _linear(self.ctx, step, h, self.w["wqkv"], "qkv", keep_partial=pos.accepts_partial_sums)
        qkv = step.ws("qkv", (step.rows, self.q_dim + 2 * self.kv_dim))
        slots = step.slots(g) if self.cache_owner else None
        attn = step.ws("attn", (step.rows, self.q_dim))
        # decode-shaped steps: rotation, page write and attention in one launch, where the position
        # encoding is a rotation by pairs (or none) and the step's shape has that kernel
        table = pos.rotation_table(step, self.hd) if pos.rotates else None
        if (table is not None or not pos.rotates) and paged_attention.attend_from_projection(
                step, ops, res, attn, kc, vc, g, self.nh, self.nkv, self.hd, self.scale, self.window, table, slots):
            return _to_residual(self.ctx, step, attn, self.w["wo"], "mixer_out")
        extra = {"source": res} if hasattr(res, "materialize") else {}
        stored = pos.apply(step, qkv, self.nh, self.nkv, self.hd,
                           cache=(kc, vc) if self.cache_owner else None, slots=slots, **extra)
        if self.cache_owner and not stored:
            ops.rope_cache(qkv, self.nh, self.nkv, self.hd, slots=slots, kcache=kc, vcache=vc,
                           block_size=self.ctx.block_size, rows=step.rows)
        paged_attention.attend(step, ops, qkv, attn, kc, vc, g, self.nh, self.nkv, self.hd, self.scale, self.window)
        return _to_residual(self.ctx, step, attn, self.w["wo"], "mixer_out")


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    """down( round(silu(gate(h))) * up(h) ) with gate and up as one fused projection
    (src/model/llama.cpp:119-122, src/cuda/kernels.cu:72-82).  params: intermediate_size."""

    capturable = True
    accepts_normed_rows = True

    def param_specs(self):
        H, I, pre = self.ctx.hidden_size, self.params["intermediate_size"], self.prefix
        return [ParamSpec("w_gate_up", ((pre + "gate_proj.weight", (I, H)), (pre + "up_proj.weight", (I, H)))),
                ParamSpec("w_down", ((pre + "down_proj.weight", (H, I)),))]

    def forward(self, step, h):
        I = self.params["intermediate_size"]
        act = step.ws("act", (step.rows, I))
        if not self.ctx.ops.gemm_swiglu(h, self.w["w_gate_up"], act):      # few rows: one launch
            h = as_tensor(h)
            if not self.ctx.ops.gemm_swiglu(h, self.w["w_gate_up"], act):
                gu = _linear(self.ctx, step, h, self.w["w_gate_up"], "gate_up")
                self.ctx.ops.swiglu(gu, act)
        return _to_residual(self.ctx, step, act, self.w["w_down"], "ffn_out")


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Embedding):
    """x = float(table[token]); nothing scaled or added (src/cuda/kernels.cu:27-32).
    params: vocab_size."""

    capturable = True

    def param_specs(self):
        return [ParamSpec("table", ((self.prefix + "weight", (self.params["vocab_size"], self.ctx.hidden_size)),),
                          role="table")]

    def forward(self, step, out):
        self.ctx.ops.embed(step.tokens, self.w["table"], out)
        return out

    def bytes_read(self, rows):
        table = self.w["table"]
        return rows * table.shape[1] * table.element_size()      # only the rows of the step's tokens

    def flops(self, rows, attended=0):
        return 0.0


@HEADS.register("linear_head")
class LinearHead(Head):
    """logits = h @ table^T in 32-bit, only for the rows that are asked for
    (src/model/llama.cpp:126-128).  params: vocab_size, tied (use the embedding's table)."""

    capturable = True

    def param_specs(self):
        if self.params.get("tied"):
            return []
        return [ParamSpec("table", ((self.prefix + "weight", (self.params["vocab_size"], self.ctx.hidden_size)),),
                          role="table")]

    def ignorable_tensors(self):
        # a tied checkpoint may still carry a copy of the shared table
        return (self.prefix + "weight",) if self.params.get("tied") else ()

    def forward(self, step, h, out):
        self.ctx.ops.gemm(h, self.w["table"], out, tuning=step.tune_products)
        return out


@BLOCKS.register("prenorm_residual")
class PreNormResidual(Block):
    """x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x))  (src/model/llama.cpp:104-124).  Each
    addition is done by the norm that follows it."""

    capturable = True

    def forward(self, step, x, pending):
        buf = step.ws("normed", (step.rows, x.shape[1]))
        n1, n2 = self.parts["norm_mixer"], self.parts["norm_ffn"]
        mixer, ffn = self.parts["mixer"], self.parts["ffn"]
        # a norm may leave its scale to the product that follows (Norm.defers) where that part takes it
        fold1 = {"defer": True} if (n1.defers and mixer.accepts_normed_rows) else {}
        fold2 = {"defer": True} if (n2.defers and ffn.accepts_normed_rows) else {}
        h = n1.forward(x, buf, add=pending if n1.accepts_partial_sums else as_tensor(pending), **fold1)
        a = mixer.forward(step, buf if h is None else h)
        h = n2.forward(x, buf, add=a if n2.accepts_partial_sums else as_tensor(a), **fold2)
        return ffn.forward(step, buf if h is None else h)
