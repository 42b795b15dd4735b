"""Python face of the native cache manager.

``CacheGroupSpec`` says what one group of layers needs; ``HostCore`` owns the native manager
(paged or contiguous policy), the scheduler that sits on it and the batch builder.  Sequences
are named by integer ids; their tokens, page tables and state slot live on the native side.
"""
import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from . import native
from .native import check, i32p, i64p, f32p, f64p, u64p

FULL_KV, WINDOW_KV, STATE = 0, 1, 2
_KIND_NAMES = {"full": FULL_KV, "window": WINDOW_KV, "state": STATE}


@dataclass(frozen=True)
class CacheGroupSpec:
    """kind: "full" (every key kept), "window" (a query at p sees keys t with p - t < window)
    or "state" (fixed-size per-request state, no pages)."""
    kind: str = "full"
    window: int = 0
    num_blocks: int = 0


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def xxh64(data: bytes, seed: int = 0) -> int:
    return native.lib().kvcm_xxh64(data, len(data), seed)


def chain_hash(parent: int, tokens) -> int:
    t = _i32(tokens)
    return native.lib().kvcm_chain_hash(parent, t.ctypes.data_as(i32p), len(t))


class BlockAllocator:
    """The page free list with reference counts, on its own (the managers embed one per group)."""

    def __init__(self, num_blocks: int):
        self._lib = native.lib()
        self._h = self._lib.kvcm_allocator_new(num_blocks)
        self.num_blocks = num_blocks

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.kvcm_allocator_delete(self._h)
            self._h = None

    def allocate(self) -> int:
        return self._lib.kvcm_allocator_allocate(self._h)

    def _op(self, op, page):
        rc = self._lib.kvcm_allocator_op(self._h, op, page)
        if rc < 0:
            raise native.HostCoreError(self._lib.kvcm_last_error().decode())
        return rc

    def free(self, page): self._op(0, page)
    def incref(self, page): self._op(1, page)
    def decref(self, page) -> bool: return bool(self._op(2, page))
    def push_free(self, page): self._op(3, page)
    def revive(self, page): self._op(4, page)
    def refcount(self, page) -> int: return self._lib.kvcm_allocator_refcount(self._h, page)
    def num_free(self) -> int: return self._lib.kvcm_allocator_num_free(self._h)


@dataclass
class SeqInfo:
    size: int
    prompt_len: int
    num_computed: int
    cached_tokens: int
    state_slot: int
    num_preemptions: int
    max_new_tokens: int
    num_hashes: int
    prefill_tokens_computed: int
    prefill_tokens_saved: int


@dataclass
class PlanEntry:
    id: int
    start: int
    count: int
    is_prefill: bool
    samples: bool
    gen_index: int
    temperature: float
    seed: int


@dataclass
class Finished:
    id: int
    prompt_len: int
    tokens: List[int]
    num_preemptions: int
    prefill_tokens_computed: int
    prefill_tokens_saved: int
    arrival: float
    admitted: float
    first_token: float
    finished: float

    @property
    def rejected(self):
        return self.first_token < 0

    @property
    def generated(self):
        return self.tokens[self.prompt_len:]


class BatchLayout:
    """Offsets (in int32 elements) of every array inside one packed metadata buffer."""
    FIELDS = ("rows", "seqs", "logit_rows", "max_context", "max_run", "total",
              "tokens", "positions", "context_lens", "row_seq", "run_start", "seq_start", "seq_end",
              "logit_row_index", "state_slots", "rows_padded", "seqs_padded", "logit_rows_padded", "sampling")
    GROUP_BASE, GROUP_STRIDE = 20, 4

    def __init__(self, desc, num_groups):
        for k, name in enumerate(self.FIELDS):
            setattr(self, name, int(desc[k]))
        self.slots = [int(desc[self.GROUP_BASE + self.GROUP_STRIDE * g]) for g in range(num_groups)]
        self.tables = [int(desc[self.GROUP_BASE + self.GROUP_STRIDE * g + 1]) for g in range(num_groups)]
        self.table_stride = [int(desc[self.GROUP_BASE + self.GROUP_STRIDE * g + 2]) for g in range(num_groups)]


class HostCore:
    def __init__(self, groups: Optional[Sequence[CacheGroupSpec]] = None, *, policy="paged", num_blocks=1024,
                 block_size=16, max_seq_len=2048, prefix_caching=False, watermark_blocks=-1,
                 watermark_frac=0.01, max_num_seqs=256, max_batched_tokens=4096, prefill_chunk=0, eos_id=-1):
        self._lib = native.lib()
        if not groups:
            groups = [CacheGroupSpec("full", 0, num_blocks)]
        self.groups = list(groups)
        if policy not in ("paged", "contiguous"):
            raise ValueError(f"unknown KV policy: {policy} (paged | contiguous)")
        kinds = _i32([_KIND_NAMES[g.kind] for g in self.groups])
        windows = _i32([g.window for g in self.groups])
        blocks = _i32([g.num_blocks for g in self.groups])
        self._h = self._lib.kvcm_core_new(
            0 if policy == "paged" else 1, len(self.groups), kinds.ctypes.data_as(i32p),
            windows.ctypes.data_as(i32p), blocks.ctypes.data_as(i32p), block_size, max_seq_len,
            int(bool(prefix_caching)), watermark_blocks, float(watermark_frac), max_num_seqs,
            max_batched_tokens, prefill_chunk, eos_id)
        if not self._h:
            raise native.HostCoreError(self._lib.kvcm_last_error().decode())
        self.policy = policy
        self.block_size = block_size
        self.max_seq_len = max_seq_len
        self.max_num_seqs = max_num_seqs
        self.max_batched_tokens = max_batched_tokens
        self.prefill_chunk = prefill_chunk
        self.prefix_caching = bool(prefix_caching) and policy == "paged"
        self._desc = np.zeros(self._lib.kvcm_batch_desc_len(self._h), dtype=np.int32)
        self._summary = np.zeros(10, dtype=np.int64)
        # of the last schedule_summary: the longest context a row of the plan sees, its rows in all, how
        # many of its first entries run one token, its longest run
        self.plan_max_context = self.plan_rows = self.plan_leading = self.plan_max_run = 0

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.kvcm_core_delete(self._h)
            self._h = None

    @property
    def name(self) -> str:
        buf = C.create_string_buffer(64)
        self._lib.kvcm_core_policy_name(self._h, buf, 64)
        return buf.value.decode()

    # ------------------------------------------------------------ sequences driven by hand
    def seq_new(self, sid, tokens, max_new_tokens=1 << 30):
        t = _i32(tokens)
        check(self._lib.kvcm_seq_new(self._h, sid, t.ctypes.data_as(i32p), len(t), max_new_tokens))

    def seq_delete(self, sid): check(self._lib.kvcm_seq_delete(self._h, sid))

    def seq_push_tokens(self, sid, tokens) -> int:
        t = _i32(tokens)
        return check(self._lib.kvcm_seq_push_tokens(self._h, sid, t.ctypes.data_as(i32p), len(t)))

    def seq_pop_token(self, sid) -> int: return check(self._lib.kvcm_seq_pop_token(self._h, sid))
    def can_admit(self, sid) -> bool: return bool(check(self._lib.kvcm_seq_can_admit(self._h, sid)))
    def admit(self, sid): check(self._lib.kvcm_seq_admit(self._h, sid))
    def append_slot(self, sid) -> bool: return bool(check(self._lib.kvcm_seq_append_slot(self._h, sid)))
    def set_computed(self, sid, n): check(self._lib.kvcm_seq_set_computed(self._h, sid, n))
    def commit(self, sid): check(self._lib.kvcm_seq_commit(self._h, sid))
    def release(self, sid): check(self._lib.kvcm_seq_release(self._h, sid))

    def seq_info(self, sid) -> SeqInfo:
        out = np.zeros(10, dtype=np.int64)
        check(self._lib.kvcm_seq_info(self._h, sid, out.ctypes.data_as(i64p)))
        return SeqInfo(*[int(v) for v in out])

    def seq_table(self, sid, group=0) -> List[int]:
        n = check(self._lib.kvcm_seq_table(self._h, sid, group, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        check(self._lib.kvcm_seq_table(self._h, sid, group, out.ctypes.data_as(i32p), n))
        return [int(v) for v in out[:n]]

    def seq_tokens(self, sid) -> List[int]:
        n = check(self._lib.kvcm_seq_tokens(self._h, sid, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        check(self._lib.kvcm_seq_tokens(self._h, sid, out.ctypes.data_as(i32p), n))
        return [int(v) for v in out[:n]]

    # --------------------------------------------------------------------- manager queries
    @property
    def num_groups(self): return len(self.groups)
    def blocks_in_use(self, g=0): return self._lib.kvcm_blocks_in_use(self._h, g)
    def blocks_cached_free(self, g=0): return self._lib.kvcm_blocks_cached_free(self._h, g)
    def state_slots_free(self): return self._lib.kvcm_state_slots_free(self._h)
    def num_free_pages(self, g=0): return check(self._lib.kvcm_num_free_pages(self._h, g))
    def page_refcount(self, page, g=0): return check(self._lib.kvcm_page_refcount(self._h, g, page))
    def num_hashed(self, g=0): return check(self._lib.kvcm_num_hashed(self._h, g))
    def num_free_extents(self, g=0): return check(self._lib.kvcm_num_free_extents(self._h, g))

    def lru_order(self, g=0) -> List[int]:
        n = check(self._lib.kvcm_lru_order(self._h, g, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        check(self._lib.kvcm_lru_order(self._h, g, out.ctypes.data_as(i32p), n))
        return [int(v) for v in out[:n]]

    def count_match(self, tokens, num_pages, g=0):
        t = _i32(tokens)
        parked = C.c_int32(0)
        hits = check(self._lib.kvcm_count_match(self._h, g, t.ctypes.data_as(i32p), num_pages, C.byref(parked)))
        return hits, parked.value

    def prefix_stats(self, g=0) -> dict:
        out = np.zeros(5, dtype=np.int64)
        self._lib.kvcm_prefix_stats(self._h, g, out.ctypes.data_as(i64p))
        keys = ("queried_blocks", "hit_blocks", "inserted_blocks", "evictions", "duplicate_inserts")
        return {k: int(v) for k, v in zip(keys, out)}

    def kv_stats(self, ids=None, g=0) -> dict:
        out = np.zeros(10, dtype=np.int64)
        if ids is None:
            check(self._lib.kvcm_kv_stats(self._h, g, None, 0, out.ctypes.data_as(i64p)))
        else:
            a = np.ascontiguousarray(np.asarray(ids, dtype=np.int64))
            check(self._lib.kvcm_kv_stats(self._h, g, a.ctypes.data_as(i64p), len(a), out.ctypes.data_as(i64p)))
        keys = ("num_blocks", "block_size", "blocks_in_use", "blocks_cached_free", "allocated_slots",
                "used_slots", "tail_waste_slots", "reserved_unused_slots", "block_table_entries", "num_seqs")
        d = {k: int(v) for k, v in zip(keys, out)}
        d["fragmentation"] = ((d["allocated_slots"] - d["used_slots"]) / d["allocated_slots"]
                              if d["allocated_slots"] else 0.0)
        return d

    # --------------------------------------------------------------------------- scheduler
    def sched_add(self, sid, tokens, max_new_tokens, temperature=0.0, sampler_seed=0, arrival=0.0):
        t = _i32(tokens)
        check(self._lib.kvcm_sched_add(self._h, sid, t.ctypes.data_as(i32p), len(t), max_new_tokens,
                                       float(temperature), int(sampler_seed) & ((1 << 64) - 1), float(arrival)))

    def schedule(self, now=0.0) -> List[PlanEntry]:
        n = check(self._lib.kvcm_sched_schedule(self._h, float(now)))
        return self.plan(n)

    def plan(self, n=None) -> List[PlanEntry]:
        cap = max(self.max_num_seqs, 1) if n is None else max(n, 1)
        ids = np.zeros(cap, dtype=np.int64)
        start, count, flags, gen = (np.zeros(cap, dtype=np.int32) for _ in range(4))
        temp = np.zeros(cap, dtype=np.float32)
        seed = np.zeros(cap, dtype=np.uint64)
        n = check(self._lib.kvcm_sched_plan(
            self._h, ids.ctypes.data_as(i64p), start.ctypes.data_as(i32p), count.ctypes.data_as(i32p),
            flags.ctypes.data_as(i32p), gen.ctypes.data_as(i32p), temp.ctypes.data_as(f32p),
            seed.ctypes.data_as(u64p), cap))
        return [PlanEntry(int(ids[k]), int(start[k]), int(count[k]), bool(flags[k] & 1), bool(flags[k] & 2),
                          int(gen[k]), float(temp[k]), int(seed[k])) for k in range(n)]

    def schedule_summary(self, now=0.0):
        """Runs the scheduler; -> (entries, prompt tokens, decoding sequences, entries that sample,
        decode_shaped) without building the plan's entries in Python (``plan()`` still gives them)."""
        check(self._lib.kvcm_sched_schedule_summary(self._h, float(now), self._summary.ctypes.data_as(i64p)))
        s = self._summary
        self.plan_max_context, self.plan_rows, self.plan_leading, self.plan_max_run = int(s[5]), int(s[6]), int(s[7]), int(s[8])
        return int(s[0]), int(s[1]), int(s[2]), int(s[3]), bool(s[4])

    def update_sampled(self, ids, now=0.0):
        """The ids sampled this step, in the order of the plan's sampling entries."""
        t = np.ascontiguousarray(ids, dtype=np.int32)
        check(self._lib.kvcm_sched_update_sampled(self._h, t.ctypes.data_as(i32p), len(t), float(now)))

    def update(self, next_tokens, now=0.0):
        t = _i32(next_tokens)
        check(self._lib.kvcm_sched_update(self._h, t.ctypes.data_as(i32p), len(t), float(now)))

    def take_finished(self) -> List[Finished]:
        n = check(self._lib.kvcm_sched_collect_finished(self._h))
        out = []
        info = np.zeros(6, dtype=np.int64)
        times = np.zeros(4, dtype=np.float64)
        for k in range(n):
            size = check(self._lib.kvcm_finished_get(self._h, k, info.ctypes.data_as(i64p),
                                                     times.ctypes.data_as(f64p), None, 0))
            toks = np.zeros(max(size, 1), dtype=np.int32)
            check(self._lib.kvcm_finished_get(self._h, k, info.ctypes.data_as(i64p),
                                              times.ctypes.data_as(f64p), toks.ctypes.data_as(i32p), size))
            out.append(Finished(int(info[0]), int(info[1]), [int(v) for v in toks[:size]], int(info[3]),
                                int(info[4]), int(info[5]), *[float(v) for v in times]))
        self._lib.kvcm_finished_clear(self._h)
        return out

    def idle(self) -> bool: return bool(self._lib.kvcm_sched_idle(self._h))
    def num_waiting(self) -> int: return self._lib.kvcm_sched_num_waiting(self._h)
    def num_running(self) -> int: return self._lib.kvcm_sched_num_running(self._h)

    def counters(self) -> dict:
        out = np.zeros(10, dtype=np.int64)
        self._lib.kvcm_sched_counters(self._h, out.ctypes.data_as(i64p))
        keys = ("steps", "preemptions", "admissions", "admission_blocked_steps", "rejected", "prefill_tokens",
                "decode_tokens", "prefill_tokens_saved", "batch_size_sum", "max_running")
        return {k: int(v) for k, v in zip(keys, out)}

    def reset_counters(self): self._lib.kvcm_sched_reset_counters(self._h)

    # ----------------------------------------------------------------------- batch builder
    def build_batch(self, entries, out: np.ndarray, *, pad_rows=0, pad_seqs=0, pad_logit_rows=0,
                    table_stride=0) -> BatchLayout:
        """entries: (id, start, count, want) with want = offsets inside the run whose logits are
        asked for, or None for "the last row".  ``out`` is a contiguous int32 array (pinned host
        memory in the engine) that receives the packed arrays."""
        n = len(entries)
        ids = np.asarray([e[0] for e in entries], dtype=np.int64)
        start = _i32([e[1] for e in entries])
        count = _i32([e[2] for e in entries])
        wants = [([e[2] - 1] if e[3] is None else list(e[3])) for e in entries]
        offs = _i32(np.concatenate([[0], np.cumsum([len(w) for w in wants])]))
        flat = _i32([w for ws in wants for w in ws] or [0])
        check(self._lib.kvcm_build_batch(
            self._h, n, ids.ctypes.data_as(i64p), start.ctypes.data_as(i32p), count.ctypes.data_as(i32p),
            offs.ctypes.data_as(i32p), flat.ctypes.data_as(i32p), pad_rows, pad_seqs, pad_logit_rows,
            table_stride, out.ctypes.data, out.size, self._desc.ctypes.data_as(i32p)))
        return BatchLayout(self._desc, self.num_groups)

    def build_batch_from_plan(self, out: np.ndarray, *, pad_rows=0, pad_seqs=0, pad_logit_rows=0,
                              table_stride=0, pad_leading=0) -> BatchLayout:
        """The scheduler's current plan as a batch.  ``pad_leading``: bring the leading single-token
        runs up to that many with padding sequences of one padding row each (recorded step shapes)."""
        check(self._lib.kvcm_build_batch_from_plan_shaped(
            self._h, pad_rows, pad_seqs, pad_logit_rows, table_stride, pad_leading, out.ctypes.data, out.size,
            self._desc.ctypes.data_as(i32p)))
        return BatchLayout(self._desc, self.num_groups)

    @property
    def handle(self):
        """The native core, for native callers (the step executor)."""
        return self._h

    def native_function(self, name) -> int:
        """Address of one of the host core's C functions."""
        return C.cast(getattr(self._lib, name), C.c_void_p).value
