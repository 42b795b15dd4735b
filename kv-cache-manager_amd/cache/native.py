"""ctypes view of libkvcm_host.so (allocator, prefix cache, managers, scheduler, batch builder)."""
import ctypes as C
import threading

from ..csrc import build as _build

_lock = threading.Lock()
_lib = None

i32p = C.POINTER(C.c_int32)
i64p = C.POINTER(C.c_int64)
u64p = C.POINTER(C.c_uint64)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)


class HostCoreError(RuntimeError):
    pass


def _declare(lib):
    def fn(name, res, *args):
        f = getattr(lib, name)
        f.restype = res
        f.argtypes = list(args)

    vp, i, i64, u64, dbl = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_double
    fn("kvcm_last_error", C.c_char_p)
    fn("kvcm_xxh64", u64, C.c_char_p, u64, u64)
    fn("kvcm_chain_hash", u64, u64, i32p, i)
    fn("kvcm_allocator_new", vp, i)
    fn("kvcm_allocator_delete", None, vp)
    fn("kvcm_allocator_allocate", i, vp)
    fn("kvcm_allocator_op", i, vp, i, i)
    fn("kvcm_allocator_refcount", i, vp, i)
    fn("kvcm_allocator_num_free", i, vp)
    fn("kvcm_core_new", vp, i, i, i32p, i32p, i32p, i, i, i, i, dbl, i, i, i, i)
    fn("kvcm_core_delete", None, vp)
    fn("kvcm_core_policy_name", i, vp, C.c_char_p, i)
    fn("kvcm_seq_new", i, vp, i64, i32p, i, i)
    fn("kvcm_seq_delete", i, vp, i64)
    fn("kvcm_seq_push_tokens", i, vp, i64, i32p, i)
    fn("kvcm_seq_pop_token", i, vp, i64)
    for name in ("can_admit", "admit", "append_slot", "commit", "release"):
        fn(f"kvcm_seq_{name}", i, vp, i64)
    fn("kvcm_seq_set_computed", i, vp, i64, i)
    fn("kvcm_seq_info", i, vp, i64, i64p)
    fn("kvcm_seq_table", i, vp, i64, i, i32p, i)
    fn("kvcm_seq_tokens", i, vp, i64, i32p, i)
    fn("kvcm_num_groups", i, vp)
    fn("kvcm_block_size", i, vp)
    for name in ("blocks_in_use", "blocks_cached_free", "num_free_pages", "num_hashed", "num_free_extents"):
        fn(f"kvcm_{name}", i, vp, i)
    fn("kvcm_state_slots_free", i, vp)
    fn("kvcm_page_refcount", i, vp, i, i)
    fn("kvcm_lru_order", i, vp, i, i32p, i)
    fn("kvcm_count_match", i, vp, i, i32p, i, i32p)
    fn("kvcm_prefix_stats", i, vp, i, i64p)
    fn("kvcm_kv_stats", i, vp, i, i64p, i, i64p)
    fn("kvcm_sched_add", i, vp, i64, i32p, i, i, C.c_float, u64, dbl)
    fn("kvcm_sched_schedule", i, vp, dbl)
    fn("kvcm_sched_plan", i, vp, i64p, i32p, i32p, i32p, i32p, f32p, u64p, i)
    fn("kvcm_sched_update", i, vp, i32p, i, dbl)
    fn("kvcm_sched_schedule_summary", i, vp, dbl, i64p)
    fn("kvcm_sched_update_sampled", i, vp, i32p, i, dbl)
    fn("kvcm_sched_collect_finished", i, vp)
    fn("kvcm_finished_get", i, vp, i, i64p, f64p, i32p, i)
    fn("kvcm_finished_clear", None, vp)
    for name in ("idle", "num_waiting", "num_running"):
        fn(f"kvcm_sched_{name}", i, vp)
    fn("kvcm_sched_counters", i, vp, i64p)
    fn("kvcm_sched_reset_counters", None, vp)
    fn("kvcm_batch_desc_len", i, vp)
    fn("kvcm_build_batch", i, vp, i, i64p, i32p, i32p, i32p, i32p, i, i, i, i, C.c_void_p, i64, i32p)
    fn("kvcm_build_batch_from_plan", i, vp, i, i, i, i, C.c_void_p, i64, i32p)
    fn("kvcm_build_batch_from_plan_shaped", i, vp, i, i, i, i, i, C.c_void_p, i64, i32p)


def lib():
    global _lib
    with _lock:
        if _lib is None:
            loaded = C.CDLL(_build.build_host())
            _declare(loaded)
            _lib = loaded
    return _lib


def check(rc):
    """Raises with the library's message when a call reported failure."""
    if rc is None or rc < 0:
        raise HostCoreError(lib().kvcm_last_error().decode())
    return rc
