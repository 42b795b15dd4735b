"""Host-side cache management: allocator, paged / contiguous managers, prefix cache, windowed
groups and state slots.  The expectations restate the reference's own CPU tests
(tests/test_block_allocator.cpp, tests/test_managers.cpp, tests/test_prefix_cache.cpp) and add
the parts the reference does not have (groups, windows, state slots)."""
import random

import pytest

from kvcm_amd.cache.manager import BlockAllocator, CacheGroupSpec, HostCore, chain_hash, xxh64
from kvcm_amd.cache.native import HostCoreError


# ------------------------------------------------------------------------------- hashing
def test_xxh64_known_vectors():
    # tests/test_prefix_cache.cpp:27-33
    assert xxh64(b"") == 0xEF46DB3751D8E999
    assert xxh64(b"a") == 0xD24EC4F1A98C6E5B
    assert xxh64(b"abc") == 0x44BC2CF5AD770999
    assert xxh64(b"Nobody inspects the spammish repetition") == 0xFBCEA83C8A378BF1


def test_chain_hash_depends_on_parent_and_tokens():
    a = chain_hash(0, [1, 2, 3, 4])
    assert a == xxh64(bytes([1, 0, 0, 0, 2, 0, 0, 0, 3, 0, 0, 0, 4, 0, 0, 0]), 0)
    assert chain_hash(a, [1, 2, 3, 4]) != a
    assert chain_hash(0, [1, 2, 3, 5]) != a


# ----------------------------------------------------------------------------- allocator
def test_allocator_allocate_all_then_free():
    a = BlockAllocator(64)
    got = [a.allocate() for _ in range(64)]
    assert got == list(range(64))          # a fresh pool hands out 0, 1, 2, ...
    assert a.allocate() == -1 and a.num_free() == 0
    for p in got:
        a.free(p)
    assert a.num_free() == 64
    assert a.allocate() == 63              # last freed, first reused


def test_allocator_refcount_keeps_page_alive_and_double_free_throws():
    a = BlockAllocator(4)
    p = a.allocate()
    a.incref(p)
    assert a.refcount(p) == 2
    a.free(p)
    assert a.num_free() == 3
    a.free(p)
    assert a.num_free() == 4
    with pytest.raises(HostCoreError):
        a.free(p)
    with pytest.raises(HostCoreError):
        a.incref(p)
    with pytest.raises(HostCoreError):
        a.push_free(p)


def test_allocator_random_cycles_no_leak_no_alias():
    # tests/test_block_allocator.cpp:37-76, same op mix with shadow reference counts
    n = 257
    a = BlockAllocator(n)
    rng = random.Random(42)
    refs = [0] * n
    live = []
    for it in range(200000):
        op = rng.randrange(3)
        if op == 0:
            p = a.allocate()
            if p < 0:
                assert live
                continue
            assert refs[p] == 0, "allocator handed out a live page"
            refs[p] = 1
            live.append(p)
        elif op == 1 and live:
            p = live[rng.randrange(len(live))]
            a.incref(p)
            refs[p] += 1
            live.append(p)
        elif live:
            k = rng.randrange(len(live))
            p = live[k]
            live[k] = live[-1]
            live.pop()
            a.free(p)
            refs[p] -= 1
        if it % 9973 == 0:
            assert a.num_free() == sum(1 for r in refs if r == 0)
            assert all(a.refcount(i) == refs[i] for i in range(n))
    for p in live:
        a.free(p)
    assert a.num_free() == n


# -------------------------------------------------------------------------------- managers
def _toks(n, base=0):
    return [3 + (base * 7919 + i * 31) % 30000 for i in range(n)]


def test_paged_allocates_on_demand():
    m = HostCore(num_blocks=100, block_size=16, max_seq_len=2048, watermark_blocks=0)
    m.seq_new(0, _toks(17))
    assert m.can_admit(0)
    m.admit(0)
    assert len(m.seq_table(0)) == 2 and m.seq_info(0).num_computed == 0 and m.blocks_in_use() == 2
    for _ in range(15):                     # fill the second page up to 32 tokens
        m.seq_push_tokens(0, [5])
        assert m.append_slot(0)
    assert len(m.seq_table(0)) == 2
    m.seq_push_tokens(0, [5])               # the 33rd token opens a third page
    assert m.append_slot(0)
    assert len(m.seq_table(0)) == 3
    m.release(0)
    assert m.blocks_in_use() == 0


def test_paged_append_fails_when_full():
    m = HostCore(num_blocks=2, block_size=4, watermark_blocks=0)
    m.seq_new(0, _toks(8))
    m.admit(0)
    m.seq_push_tokens(0, [1])
    assert not m.append_slot(0)
    m.seq_new(1, [1])
    assert not m.can_admit(1)


def test_watermark_keeps_pages_spare_at_admission():
    m = HostCore(num_blocks=100, block_size=16, watermark_frac=0.05)   # 5 pages spare
    m.seq_new(0, _toks(16 * 95))
    assert m.can_admit(0)
    m.seq_new(1, _toks(16 * 96))
    assert not m.can_admit(1)


def test_too_long_is_never_admitted():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=64)
    m.seq_new(0, _toks(65))
    assert not m.can_admit(0)


def test_contiguous_reserves_max_seq_len():
    m = HostCore(policy="contiguous", num_blocks=64, block_size=16, max_seq_len=256)  # 16 pages each
    for i in range(5):
        m.seq_new(i, _toks(5, i))
    for i in range(4):
        assert m.can_admit(i)
        m.admit(i)
        t = m.seq_table(i)
        assert len(t) == 16 and all(t[k] == t[k - 1] + 1 for k in range(1, 16))
    assert not m.can_admit(4)               # only four fit although each holds five tokens
    m.release(1)
    assert m.can_admit(4)
    for i in (0, 2, 3):
        m.release(i)
    assert m.blocks_in_use() == 0 and m.num_free_extents() == 1


def test_contiguous_external_fragmentation():
    m = HostCore(policy="contiguous", num_blocks=48, block_size=16, max_seq_len=256)
    for i in range(3):
        m.seq_new(i, _toks(5, i))
        m.admit(i)
    m.release(0)
    m.release(2)
    assert m.num_free_extents() == 2
    m.release(1)
    assert m.num_free_extents() == 1


@pytest.mark.parametrize("policy,seed", [("paged", 1), ("contiguous", 2)])
def test_random_churn_no_alias_no_leak(policy, seed):
    # tests/test_managers.cpp:87-138
    m = HostCore(policy=policy, num_blocks=512, block_size=16, max_seq_len=1024, watermark_blocks=0)
    rng = random.Random(seed)
    live = {}
    next_id = 0
    for it in range(6000):
        op = rng.randrange(4)
        if op == 0:
            n = 1 + rng.randrange(300)
            m.seq_new(next_id, _toks(n, next_id))
            if m.can_admit(next_id):
                m.admit(next_id)
                m.set_computed(next_id, n)
                live[next_id] = n
            else:
                m.seq_delete(next_id)
            next_id += 1
        elif op <= 2 and live:
            sid = rng.choice(list(live))
            if live[sid] < m.max_seq_len:
                m.seq_push_tokens(sid, [7])
                if m.append_slot(sid):
                    live[sid] += 1
                    m.set_computed(sid, live[sid])
                else:
                    m.seq_pop_token(sid)
        elif live:
            sid = rng.choice(list(live))
            m.release(sid)
            m.seq_delete(sid)
            del live[sid]
        if it % 50 == 0:
            owned = set()
            total = 0
            for sid, n in live.items():
                t = m.seq_table(sid)
                assert len(t) * 16 >= n
                for p in t:
                    assert p not in owned, f"page {p} held twice"
                    owned.add(p)
                total += len(t)
            assert m.blocks_in_use() == total
            assert m.state_slots_free() == 256 - len(live)
    for sid in live:
        m.release(sid)
    assert m.blocks_in_use() == 0 and m.state_slots_free() == 256


def test_kv_stats_fragmentation_accounting():
    p = HostCore(num_blocks=100, block_size=16, max_seq_len=256)
    c = HostCore(policy="contiguous", num_blocks=100, block_size=16, max_seq_len=256)
    for m in (p, c):
        m.seq_new(0, _toks(20))
        m.admit(0)
        m.set_computed(0, 20)
    sp, sc = p.kv_stats([0]), c.kv_stats([0])
    assert (sp["allocated_slots"], sp["used_slots"], sp["tail_waste_slots"], sp["reserved_unused_slots"]) == (32, 20, 12, 0)
    assert (sc["allocated_slots"], sc["used_slots"], sc["tail_waste_slots"], sc["reserved_unused_slots"]) == (256, 20, 12, 224)


# ---------------------------------------------------------------------------- prefix cache
def _computed(m, sid):
    m.set_computed(sid, m.seq_info(sid).size)
    m.commit(sid)


def test_prefix_hit_and_miss():
    m = HostCore(num_blocks=32, block_size=4, max_seq_len=256, prefix_caching=True, watermark_blocks=0)
    base = list(range(100, 113))
    m.seq_new(0, base)
    m.admit(0)
    assert m.seq_info(0).num_computed == 0
    _computed(m, 0)
    assert m.num_hashed() == 3
    m.seq_new(1, base)
    assert m.can_admit(1)
    m.admit(1)
    i1 = m.seq_info(1)
    assert i1.cached_tokens == 12 and i1.num_computed == 12
    ta, tb = m.seq_table(0), m.seq_table(1)
    for k in range(3):
        assert tb[k] == ta[k] and m.page_refcount(ta[k]) == 2
    assert tb[3] != ta[3]                    # the tail stays private
    t = list(base)
    t[5] = 9999                              # shares the first page only
    m.seq_new(2, t)
    m.admit(2)
    assert m.seq_info(2).cached_tokens == 4 and m.seq_table(2)[0] == ta[0]
    t = list(base)
    t[0] = 1                                 # another first page: nothing hits
    m.seq_new(3, t)
    m.admit(3)
    assert m.seq_info(3).cached_tokens == 0
    st = m.prefix_stats()
    assert st["hit_blocks"] == 4 and st["queried_blocks"] == 12


def test_prefix_full_hit_still_recomputes_last_token():
    m = HostCore(num_blocks=32, block_size=4, prefix_caching=True, watermark_blocks=0)
    m.seq_new(0, list(range(8)))
    m.admit(0)
    _computed(m, 0)
    assert m.num_hashed() == 2
    m.seq_new(1, list(range(8)))
    m.admit(1)
    assert m.seq_info(1).cached_tokens == 4 and m.seq_table(1)[1] != m.seq_table(0)[1]


def test_released_pages_stay_findable():
    m = HostCore(num_blocks=16, block_size=4, prefix_caching=True, watermark_blocks=0)
    m.seq_new(0, list(range(13)))
    m.admit(0)
    _computed(m, 0)
    pages = m.seq_table(0)
    m.release(0)
    assert m.blocks_in_use() == 0 and m.blocks_cached_free() == 3
    m.seq_new(1, list(range(13)))
    assert m.can_admit(1)
    m.admit(1)
    assert m.seq_info(1).cached_tokens == 12 and m.seq_table(1)[:3] == pages[:3]
    assert m.blocks_cached_free() == 0


def test_eviction_is_lru_and_tail_first():
    m = HostCore(num_blocks=8, block_size=4, prefix_caching=True, watermark_blocks=0)
    m.seq_new(0, list(range(9)))
    m.seq_new(1, list(range(500, 509)))
    for s in (0, 1):
        m.admit(s)
        _computed(m, s)
    xb, yb = m.seq_table(0), m.seq_table(1)
    m.release(0)
    m.release(1)
    assert m.lru_order() == [xb[1], xb[0], yb[1], yb[0]]
    assert m.num_free_pages() == 4
    m.seq_new(2, list(range(9000, 9020)))    # five pages: one eviction, x's tail goes first
    assert m.can_admit(2)
    m.admit(2)
    assert m.prefix_stats()["evictions"] == 1
    assert m.lru_order() == [xb[0], yb[1], yb[0]]
    assert m.count_match(list(range(9)), 2) == (1, 1)


def test_can_admit_accounts_for_lru_hits():
    m = HostCore(num_blocks=4, block_size=4, prefix_caching=True, watermark_blocks=0)
    m.seq_new(0, list(range(9)))
    m.admit(0)
    _computed(m, 0)
    m.release(0)
    m.seq_new(1, list(range(16)))            # 2 hits + 2 fresh pages: fits exactly
    assert m.can_admit(1)
    m.seq_new(2, list(range(17)))            # 2 hits + 3 fresh
    assert not m.can_admit(2)


def test_prefix_disabled_never_caches():
    m = HostCore(num_blocks=16, block_size=4, prefix_caching=False, watermark_blocks=0)
    for s in (0, 1):
        m.seq_new(s, list(range(13)))
        m.admit(s)
        _computed(m, s)
    assert m.seq_info(1).cached_tokens == 0
    m.release(0)
    m.release(1)
    assert m.num_free_pages() == 16


def test_contiguous_policy_turns_prefix_caching_off():
    m = HostCore(policy="contiguous", num_blocks=64, block_size=4, max_seq_len=32, prefix_caching=True)
    assert m.prefix_caching is False and m.name == "contiguous"


# ------------------------------------------------------------- groups, windows, state slots
def test_groups_have_pages_of_their_own():
    groups = [CacheGroupSpec("full", 0, 40), CacheGroupSpec("window", 8, 10), CacheGroupSpec("state")]
    m = HostCore(groups, block_size=4, max_seq_len=200, watermark_blocks=0, max_num_seqs=3)
    m.seq_new(0, _toks(10))
    m.admit(0)
    assert len(m.seq_table(0, 0)) == 3 and len(m.seq_table(0, 1)) == 3 and m.seq_table(0, 2) == []
    assert m.blocks_in_use(0) == 3 and m.blocks_in_use(1) == 3 and m.blocks_in_use(2) == 0
    assert m.seq_info(0).state_slot == 0
    m.release(0)
    assert m.blocks_in_use(0) == 0 and m.blocks_in_use(1) == 0 and m.state_slots_free() == 3


def test_window_gives_pages_back_once_passed():
    # window 8, page 4: a query at position p sees keys p-7..p
    groups = [CacheGroupSpec("full", 0, 64), CacheGroupSpec("window", 8, 6)]
    m = HostCore(groups, block_size=4, max_seq_len=200, watermark_blocks=0)
    m.seq_new(0, _toks(9))
    m.admit(0)
    m.set_computed(0, 9)
    m.commit(0)                              # next query at 9 sees keys >= 2: page 0 still needed
    assert m.seq_table(0, 1) == [0, 1, 2]
    freed = []
    for n in range(10, 60):
        m.seq_push_tokens(0, [7])
        assert m.append_slot(0), "the small window pool must suffice because pages come back"
        m.set_computed(0, n)
        m.commit(0)
        t = m.seq_table(0, 1)
        first_needed = max(0, n - 8 + 1) // 4
        assert all(p == -1 for p in t[:first_needed]) and all(p >= 0 for p in t[first_needed:])
        freed.append(first_needed)
        assert m.blocks_in_use(1) == len(t) - first_needed <= 4
        assert all(p >= 0 for p in m.seq_table(0, 0))   # the full group keeps everything
    assert freed[-1] > 5
    m.release(0)
    assert m.blocks_in_use(0) == 0 and m.blocks_in_use(1) == 0 and m.num_free_pages(1) == 6


def test_prefix_caching_refuses_windows_and_state():
    with pytest.raises(HostCoreError, match="prefix caching"):
        HostCore([CacheGroupSpec("window", 8, 10)], block_size=4, prefix_caching=True)
    with pytest.raises(HostCoreError, match="prefix caching"):
        HostCore([CacheGroupSpec("full", 0, 10), CacheGroupSpec("state")], block_size=4, prefix_caching=True)


def test_state_slots_limit_admission_and_are_not_returned_twice():
    m = HostCore([CacheGroupSpec("full", 0, 100), CacheGroupSpec("state")], block_size=4, max_num_seqs=2,
                 watermark_blocks=0)
    for s in range(3):
        m.seq_new(s, _toks(5, s))
    m.admit(0)
    m.admit(1)
    assert {m.seq_info(0).state_slot, m.seq_info(1).state_slot} == {0, 1}
    assert not m.can_admit(2)
    m.release(0)
    m.release(0)                              # releasing twice is harmless: nothing is held
    assert m.state_slots_free() == 1 and m.can_admit(2)
    m.admit(2)
    assert m.seq_info(2).state_slot == 0      # the slot is used again
    with pytest.raises(HostCoreError):
        m.admit(2)


def test_random_orders_with_groups_never_lose_a_page():
    groups = [CacheGroupSpec("full", 0, 96), CacheGroupSpec("window", 12, 48), CacheGroupSpec("state")]
    m = HostCore(groups, block_size=4, max_seq_len=160, watermark_blocks=0, max_num_seqs=8)
    rng = random.Random(7)
    live = {}
    nid = 0
    for it in range(4000):
        op = rng.randrange(5)
        if op == 0:
            n = 1 + rng.randrange(60)
            m.seq_new(nid, _toks(n, nid))
            if m.can_admit(nid):
                m.admit(nid)
                m.set_computed(nid, n)
                m.commit(nid)
                live[nid] = n
            else:
                m.seq_delete(nid)
            nid += 1
        elif op <= 3 and live:
            sid = rng.choice(list(live))
            if live[sid] < 160:
                m.seq_push_tokens(sid, [9])
                if m.append_slot(sid):
                    live[sid] += 1
                    m.set_computed(sid, live[sid])
                    m.commit(sid)
                else:
                    m.seq_pop_token(sid)
        elif live:
            sid = rng.choice(list(live))
            m.release(sid)
            m.seq_delete(sid)
            del live[sid]
        if it % 40 == 0:
            for g in (0, 1):
                held = [p for sid in live for p in m.seq_table(sid, g) if p >= 0]
                assert len(held) == len(set(held)), "a page is held twice"
                assert m.blocks_in_use(g) == len(held)
                assert m.num_free_pages(g) == groups[g].num_blocks - len(held), "a page was lost"
            slots = [m.seq_info(sid).state_slot for sid in live]
            assert len(set(slots)) == len(slots) and m.state_slots_free() == 8 - len(live)
    for sid in list(live):
        m.release(sid)
    assert m.num_free_pages(0) == 96 and m.num_free_pages(1) == 48 and m.state_slots_free() == 8


def test_storage_refuses_a_cache_beyond_the_kernels_addressing():
    """Slot numbers are 32-bit and the decode kernels keep offsets inside a layer's cache in 32
    bits (units of 8 elements): a pool beyond that is refused when it is made, not at its first step."""
    import torch
    from kvcm_amd.cache.storage import KVStorage
    from kvcm_amd.parts.base import KVCacheNeed
    ok = KVStorage(0, KVCacheNeed(8, 128), 2, 2 ** 21, 16, torch.bfloat16, "meta")       # 2^35 elements per layer
    assert ok.k(1).shape == (2 ** 21, 8, 16, 128)
    with pytest.raises(ValueError, match="more than the kernels address"):
        KVStorage(0, KVCacheNeed(8, 128), 2, 2 ** 21 + 1, 16, torch.bfloat16, "meta")
    with pytest.raises(ValueError, match="more than the kernels address"):
        KVStorage(0, KVCacheNeed(1, 8), 1, 2 ** 27, 16, torch.bfloat16, "meta")             # 2^31 token slots
