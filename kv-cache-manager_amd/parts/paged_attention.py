"""Which attention kernel a step takes: shared by every mixer that attends over paged keys and
values.  It uses nothing of the step beyond what parts.base.StepView declares, so a second
attention-like mixer calls these two functions (or picks kernels from ``ctx.ops`` itself) without
the engine changing.

  attend                   q is rotated and the step's keys and values are in their pages already
  attend_from_projection   from the fused [q | k | v] projection (finished rows or un-added split-K
                           sums) to the attention output: rotation, page write and attention in one
                           launch where the step's shape and the head shape have such a kernel

The reference picks between its one-pass and its partitioned kernel in the same place
(src/cuda/paged_attention.cu:353-371, option --attn).
"""
import torch

# Rows up to which a step of single-token runs is treated as decode-shaped.
DECODE_ATTENTION_MAX_ROWS = 512


def _decode_parts_scratch(step, ops, rows, nh, nkv, hd, bound):
    """Scratch for the decode kernel when it cuts long contexts of few rows into parts; sized at
    once for the worst case (rows x parts <= 256 / kv heads + rows), so that a recorded step's
    pointer stays good."""
    need = ops.attention_decode_fused_scratch(rows, nh, nkv, hd, bound)
    if need == 0:
        return None
    most_rows = min(DECODE_ATTENTION_MAX_ROWS, step.limits.max_tokens)
    worst = nh * (256 // nkv + 1 + most_rows) * (hd + 2)
    return step.flat("decode_parts", max(need, worst))


def attend_from_projection(step, ops, projection, out, kcache, vcache, g, nh, nkv, hd, scale, window, cos_sin, slots):
    """Decode-shaped steps: one launch (and a small merge when few rows have long contexts).  Steps
    with runs of positions: the keys of those rows are rotated and stored with their values, the tiled
    kernel rotates their queries as it reads them; where the first sequences of such a step run one
    token each (the scheduler puts decoding requests first) those rows take the decode launch: a
    single-token run would otherwise cost a whole tile of its own.
    Returns False when this step or shape has no such kernel (then the caller rotates, stores and
    calls ``attend``: the same values up to rounding)."""
    if (step.attention_mode != "auto" or window != 0 or out.dtype != torch.bfloat16
            or not ops.attention_decode_fused_supported(nh, nkv, hd, out.dtype, kcache.shape[2])):
        return False
    if step.max_run == 1:
        if step.rows > DECODE_ATTENTION_MAX_ROWS:
            return False
        bound = step.max_context_bound
        ops.attention_decode_fused(projection, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                                   step.ctx_lens, nh, nkv, hd, scale, cos_sin=cos_sin, slots=slots, rows=step.rows,
                                   max_context=bound, scratch=_decode_parts_scratch(step, ops, step.rows, nh, nkv, hd, bound))
        return True
    D, T, S = step.leading_single_runs(), step.real_rows, step.real_seqs
    if D > DECODE_ATTENTION_MAX_ROWS or not ops.attention_prefill_supported(nh, nkv, hd, out.dtype, kcache.shape[2]):
        return False
    if isinstance(projection, ops.PartialSums):
        # several consumers here (decode rows, rotation of the others, tiled attention): add the
        # split sums up once instead of handing every single-token run to the tiled kernel
        projection = projection.materialize()
    stride = step.table_stride(g)
    bound = step.max_context_bound
    if D > 0:
        ops.attention_decode_fused(projection, out, kcache, vcache, step.tables(g), stride, step.row_seq, step.ctx_lens,
                                   nh, nkv, hd, scale, cos_sin=cos_sin, slots=slots, rows=D, max_context=bound,
                                   scratch=_decode_parts_scratch(step, ops, D, nh, nkv, hd, bound))
    # the other rows: their keys are rotated and stored with their values; their queries stay as the
    # projection left them and the tiled kernel rotates them as it reads them (one pass over q less)
    if (cos_sin is not None or slots is not None) and T > D:
        ops.rope_cache(projection[D:T], nh, nkv, hd, cos_sin=cos_sin[D:T] if cos_sin is not None else None,
                       slots=slots[D:T] if slots is not None else None, kcache=kcache, vcache=vcache,
                       block_size=kcache.shape[2], rows=T - D, skip_q=True)
    need = ops.attention_prefill_scratch(T, nh, hd, bound, step.max_run, S - D)
    scratch = step.flat("prefill_partials", need) if need else None
    ops.attention_prefill(projection, out, kcache, vcache, step.tables(g)[D * stride:], stride, step.run_start[D:],
                          step.seq_start[D:], S - D, step.max_run, nh, nkv, hd, scale, rows=T,
                          max_context=bound, scratch=scratch, cos_sin=cos_sin)
    return True


def attend(step, ops, q, out, kcache, vcache, g, nh, nkv, hd, scale, window=0):
    """attention_mode "v1": the generic kernel, one pass over the whole context per (row, head);
    "v2" and "auto": for bfloat16, decode-shaped steps take the kernel that cuts contexts into
    partitions and merges them, steps with runs of positions take the tiled kernel; "v2" insists
    on the partitioned kernel for decode steps.  The 32-bit path always takes v1, whose result does
    not depend on the batch."""
    mode = step.attention_mode
    partitioned = (mode != "v1" and window == 0 and step.max_run == 1 and step.rows <= DECODE_ATTENTION_MAX_ROWS
                   and ops.attention_decode_supported(nh, nkv, hd, q.dtype, kcache.shape[2]))
    if mode == "v2" and not partitioned and q.dtype == torch.bfloat16 and step.max_run == 1:
        raise RuntimeError(f"attn=v2: the partitioned kernel does not take heads={nh} kv_heads={nkv} "
                           f"head_dim={hd} window={window} rows={step.rows}")
    if partitioned:
        bound = step.max_context_bound
        need = ops.attention_decode_scratch(step.rows, nh, hd, bound)
        scratch = step.flat("attention_partials", max(need, ops.attention_decode_scratch(
            min(DECODE_ATTENTION_MAX_ROWS, step.limits.max_tokens), nh, hd, step.limits.max_context_len)))
        ops.attention_decode(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                             step.ctx_lens, nh, nkv, hd, scale, bound, scratch, rows=step.rows)
        return
    if (mode != "v1" and window == 0 and step.max_run > 1
            and ops.attention_prefill_supported(nh, nkv, hd, q.dtype, kcache.shape[2])):
        # runs of consecutive positions: keys are read once per 64 query rows, on the matrix cores
        bound = step.max_context_bound
        need = ops.attention_prefill_scratch(step.real_rows, nh, hd, bound, step.max_run, step.real_seqs)
        scratch = step.flat("prefill_partials", need) if need else None
        ops.attention_prefill(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.run_start,
                              step.seq_start, step.real_seqs, step.max_run, nh, nkv, hd, scale,
                              rows=step.real_rows, max_context=bound, scratch=scratch)
        return
    ops.attention(q, out, kcache, vcache, step.tables(g), step.table_stride(g), step.row_seq,
                  step.ctx_lens, nh, nkv, hd, scale, window, rows=step.rows)
