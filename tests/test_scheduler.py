"""The scheduler's decisions with a fake model (every sampled token is 42), as the reference
tests them (tests/test_scheduler.cpp), plus portions of prompts under a token budget."""
import numpy as np
import pytest
from kvcm_amd.cache.manager import HostCore


def _prompt(i, n):
    return [10 + (i * 131 + k) % 1000 for k in range(n)]


def run_to_completion(m, max_steps=100000, check_whole=True):
    steps, done = 0, []
    while not m.idle() and steps < max_steps:
        plan = m.schedule(steps)
        for p in plan:
            # every scheduled run has pages for all the tokens it computes
            assert len(m.seq_table(p.id)) * m.block_size >= p.start + p.count
            if check_whole:
                assert p.start + p.count == m.seq_info(p.id).size and p.samples
        m.update([42] * len(plan), steps + 1)
        for f in m.take_finished():
            done.append(f)
        steps += 1
    return done, steps


def test_completes_all_without_pressure():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=1024)
    for i in range(20):
        m.sched_add(i, _prompt(i, 30 + i), 10 + i)
    done, _ = run_to_completion(m)
    assert len(done) == 20
    for f in done:
        assert len(f.generated) == 10 + f.id and f.generated == [42] * (10 + f.id)
    assert m.counters()["preemptions"] == 0 and m.blocks_in_use() == 0


def test_preempts_under_pressure_and_still_finishes():
    # 24 pages of 16 = 384 slots; 8 requests of 32 + 64 = 96 tokens each
    m = HostCore(num_blocks=24, block_size=16, max_seq_len=1024)
    for i in range(8):
        m.sched_add(i, _prompt(i, 32), 64)
    done, _ = run_to_completion(m)
    assert len(done) == 8 and all(len(f.generated) == 64 for f in done)
    assert m.counters()["preemptions"] > 0
    assert any(f.num_preemptions > 0 for f in done)
    assert m.blocks_in_use() == 0 and m.state_slots_free() == 256


def test_preemption_takes_the_youngest_and_puts_it_first_in_line():
    m = HostCore(num_blocks=4, block_size=4, max_seq_len=64, watermark_blocks=0)
    m.sched_add(0, _prompt(0, 7), 5)        # two pages
    m.sched_add(1, _prompt(1, 7), 5)        # two pages: the pool is full
    plan = m.schedule(0)
    assert [p.id for p in plan] == [0, 1]
    m.update([42, 42], 0)                    # both now hold 8 tokens = 2 full pages
    assert [p.id for p in m.schedule(1)] == [0, 1]
    m.update([42, 42], 1)                    # 9 tokens each: both want a third page
    plan = m.schedule(2)                     # request 0 asks first: 1 (the youngest) is preempted
    assert [p.id for p in plan] == [0]
    assert m.counters()["preemptions"] == 1 and m.num_waiting() == 1 and m.num_running() == 1
    assert m.seq_info(1).num_computed == 0 and m.seq_info(1).size == 9   # its tokens are kept
    m.update([42], 2)
    done, _ = run_to_completion(m)
    assert sorted(f.id for f in done) == [0, 1] and all(len(f.generated) == 5 for f in done)


def test_prefix_caching_skips_prefill():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=1024, prefix_caching=True)
    m.sched_add(0, _prompt(0, 100), 5)
    run_to_completion(m)
    m.sched_add(1, _prompt(0, 100), 5)       # the same prompt again
    plan = m.schedule(0)
    assert len(plan) == 1 and plan[0].start == 96 and plan[0].count == 4   # six full pages cached
    assert m.counters()["prefill_tokens_saved"] == 96


def test_rejects_impossible_requests_and_serves_the_next():
    m = HostCore(num_blocks=4, block_size=16, max_seq_len=1024)   # 64 slots in all
    m.sched_add(0, _prompt(0, 200), 5)
    m.sched_add(1, _prompt(1, 10), 5)
    done, _ = run_to_completion(m, max_steps=100)
    assert len(done) == 2 and m.counters()["rejected"] == 1
    by_id = {f.id: f for f in done}
    assert by_id[0].rejected and by_id[0].generated == []
    assert not by_id[1].rejected and len(by_id[1].generated) == 5


def test_token_budget_stops_admission_but_never_starves():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=4096, max_batched_tokens=100)
    m.sched_add(0, _prompt(0, 300), 2)       # larger than the whole budget: admitted when the step is empty
    m.sched_add(1, _prompt(1, 60), 2)
    m.sched_add(2, _prompt(2, 60), 2)
    plan = m.schedule(0)
    assert [(p.id, p.count) for p in plan] == [(0, 300)]
    m.update([42], 0)
    plan = m.schedule(1)                     # decode of 0 (1 token) + 60 fits, the next 60 does not
    assert [(p.id, p.count) for p in plan] == [(0, 1), (1, 60)]


def test_max_num_seqs_limits_running():
    m = HostCore(num_blocks=1000, block_size=16, max_num_seqs=3)
    for i in range(7):
        m.sched_add(i, _prompt(i, 5), 4)
    plan = m.schedule(0)
    assert len(plan) == 3 and m.num_waiting() == 4
    m.update([42] * 3, 0)
    done, _ = run_to_completion(m)
    assert len(done) == 7 and m.counters()["max_running"] == 3


def test_finishes_at_max_seq_len_and_at_eos():
    m = HostCore(num_blocks=100, block_size=4, max_seq_len=12)
    m.sched_add(0, _prompt(0, 8), 100)
    done, _ = run_to_completion(m)
    assert len(done[0].tokens) == 12         # the last sampled token is appended but never run
    m = HostCore(num_blocks=100, block_size=4, max_seq_len=64, eos_id=42)
    m.sched_add(0, _prompt(0, 8), 100)
    done, _ = run_to_completion(m)
    assert done[0].generated == [42]


# ----------------------------------------------------------------------- portions of prompts
def test_chunking_cuts_prompts_under_the_budget():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=4096, max_batched_tokens=64, prefill_chunk=48)
    m.sched_add(0, _prompt(0, 100), 3)
    m.sched_add(1, _prompt(1, 30), 3)
    seen = {0: [], 1: []}
    sampled = {0: 0, 1: 0}
    steps = 0
    while not m.idle():
        plan = m.schedule(steps)
        assert sum(p.count for p in plan) <= 64
        for p in plan:
            info = m.seq_info(p.id)
            assert p.start == info.num_computed          # portions are consecutive and in order
            assert p.count <= 48 or not p.is_prefill
            assert p.samples == (p.start + p.count == info.size)
            seen[p.id].append((p.start, p.count))
            sampled[p.id] += p.samples
        sizes = {p.id: m.seq_info(p.id).size for p in plan}
        m.update([42] * len(plan), steps)
        for p in plan:
            if not p.samples:                            # no token for an unfinished portion
                assert m.seq_info(p.id).size == sizes[p.id]
        m.take_finished()
        steps += 1
    assert sum(c for s, c in seen[0] if s < 100) == 100 and sum(c for s, c in seen[1] if s < 30) == 30
    assert seen[0][0] == (0, 48)
    assert sampled == {0: 3, 1: 3}


def test_chunked_first_step_shares_budget_in_arrival_order():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=4096, max_batched_tokens=64, prefill_chunk=48)
    m.sched_add(0, _prompt(0, 100), 3)
    m.sched_add(1, _prompt(1, 30), 3)
    plan = m.schedule(0)
    assert [(p.id, p.start, p.count, p.samples) for p in plan] == [(0, 0, 48, False), (1, 0, 16, False)]
    m.update([42, 42], 0)
    assert m.seq_info(0).size == 100 and m.seq_info(1).size == 30
    plan = m.schedule(1)
    assert [(p.id, p.start, p.count, p.samples) for p in plan] == [(0, 48, 48, False), (1, 16, 14, True)]
    m.update([42, 42], 1)
    assert m.seq_info(1).size == 31
    plan = m.schedule(2)                     # decode of 1 first in the budget, then the rest of 0
    assert [(p.id, p.start, p.count, p.samples) for p in plan] == [(0, 96, 4, True), (1, 30, 1, True)]


def test_chunking_off_equals_whole_prompts():
    def trace(chunk):
        m = HostCore(num_blocks=64, block_size=16, max_seq_len=1024, prefill_chunk=chunk)
        for i in range(6):
            m.sched_add(i, _prompt(i, 20 + 9 * i), 12)
        out, steps = [], 0
        while not m.idle():
            plan = m.schedule(steps)
            out.append([(p.id, p.start, p.count) for p in plan])
            m.update([42] * len(plan), steps)
            m.take_finished()
            steps += 1
        return out
    whole = trace(0)
    assert all(s + c > 0 for step in whole for _, s, c in step)
    assert trace(1 << 20) == whole           # a chunk larger than any prompt changes nothing


def test_chunked_preemption_recomputes_and_finishes():
    m = HostCore(num_blocks=20, block_size=4, max_seq_len=256, max_batched_tokens=16, prefill_chunk=8,
                 watermark_blocks=0)
    for i in range(5):
        m.sched_add(i, _prompt(i, 14), 30)
    done, steps = run_to_completion(m, check_whole=False)
    assert len(done) == 5 and all(len(f.generated) == 30 for f in done)
    assert m.counters()["preemptions"] > 0 and m.blocks_in_use() == 0


def test_plan_batch_carries_sampling_parameters_for_every_logit_row():
    core = HostCore(num_blocks=32, block_size=4, max_seq_len=64, max_num_seqs=8, max_batched_tokens=64)
    big = (1 << 63) + 12345                                  # a seed beyond the signed range keeps its bits
    core.sched_add(7, [1, 2, 3], 4, temperature=0.5, sampler_seed=big)
    core.sched_add(9, [4, 5, 6, 7, 8], 4, temperature=0.0, sampler_seed=3)
    plan = core.schedule()
    assert [p.id for p in plan] == [7, 9]
    out = np.full(4096, 77, dtype=np.int32)
    L = core.build_batch_from_plan(out, pad_logit_rows=4)
    R = L.logit_rows_padded
    assert L.logit_rows == 2 and R == 4 and L.sampling % 2 == 0 and L.sampling + 6 * R <= L.total
    o = L.sampling
    np.testing.assert_array_equal(out[o:o + R].view(np.float32), [0.5, 0.0, 0.0, 0.0])
    np.testing.assert_array_equal(out[o + R:o + 2 * R], [0, 0, 0, 0])                    # index of the token to draw
    np.testing.assert_array_equal(out[o + 2 * R:o + 4 * R].view(np.uint64), [big, 3, 0, 0])
    np.testing.assert_array_equal(out[o + 4 * R:o + 6 * R].view(np.int64), [7, 9, 0, 0])
    core.update([11, 12])
    core.schedule()
    L = core.build_batch_from_plan(out)
    o, R = L.sampling, L.logit_rows_padded
    np.testing.assert_array_equal(out[o + R:o + 2 * R], [1, 1])                          # second generated token


def test_schedule_summary_and_update_by_sampled_ids():
    core = HostCore(num_blocks=64, block_size=4, max_seq_len=64, max_num_seqs=8, max_batched_tokens=64, prefill_chunk=4)
    core.sched_add(1, [5, 6, 7], 3)              # fits one portion: samples in the first step
    core.sched_add(2, list(range(10, 19)), 3)    # 9 tokens: three portions, samples in the third
    n, prefill, decode, sampling, shaped = core.schedule_summary()
    assert (n, prefill, decode, sampling, shaped) == (2, 7, 0, 1, False)
    assert core.plan_max_context == 4            # the longest context a row of this plan sees: tokens 0..3 of request 2
    assert [(p.id, p.count, p.samples) for p in core.plan()] == [(1, 3, True), (2, 4, False)]
    with pytest.raises(Exception):
        core.update_sampled([42, 43])            # one sampling entry, two ids
    core.update_sampled([42])
    n, prefill, decode, sampling, shaped = core.schedule_summary()
    assert (n, prefill, decode, sampling, shaped) == (2, 4, 1, 1, False)       # request 1 decodes beside a portion of 2
    core.update_sampled([43])
    n, prefill, decode, sampling, shaped = core.schedule_summary()
    assert (n, prefill, decode, sampling, shaped) == (2, 1, 1, 2, True)        # a prompt's last single token: shaped like a decode, booked as prompt
    assert core.plan_max_context == 9            # request 2's ninth token
    core.update_sampled([44, 50])
    n, prefill, decode, sampling, shaped = core.schedule_summary()
    assert (n, prefill, decode, sampling, shaped) == (1, 0, 1, 1, True)        # request 1 is done, request 2 decodes
    core.update_sampled([51])
    done = {f.id: f.generated for f in core.take_finished()}
    assert done[1] == [42, 43, 44]


def test_a_prompt_whose_last_portion_is_one_token_is_still_booked_as_prompt():
    m = HostCore(num_blocks=100, block_size=4, max_seq_len=64, prefill_chunk=6)
    m.sched_add(0, _prompt(0, 7), 3)
    kinds = []
    while not m.idle():
        plan = m.schedule(0)
        kinds.append([(p.start, p.count, p.is_prefill, p.samples) for p in plan])
        m.update([42] * len(plan), 0)
    assert kinds == [[(0, 6, True, False)], [(6, 1, True, True)], [(7, 1, False, True)], [(8, 1, False, True)]]
    c = m.counters()
    assert c["prefill_tokens"] == 7 and c["decode_tokens"] == 2      # the third sampled token is never run
    f = m.take_finished()[0]
    assert f.prefill_tokens_computed == 7 and len(f.generated) == 3


def test_an_uncut_prompt_larger_than_the_budget_runs_whole_in_an_empty_step():
    m = HostCore(num_blocks=1000, block_size=16, max_seq_len=4096, max_batched_tokens=100)
    m.sched_add(0, _prompt(0, 300), 2)
    m.sched_add(1, _prompt(1, 40), 2)
    plan = m.schedule(0)
    assert [(p.id, p.start, p.count, p.samples) for p in plan] == [(0, 0, 300, True)]       # not cut, and nothing beside it
    m.update([42], 0)
    plan = m.schedule(1)
    assert [(p.id, p.start, p.count) for p in plan] == [(0, 300, 1), (1, 0, 40)]


def test_batch_padded_to_a_recorded_shape_puts_padding_sequences_after_the_leading_single_rows():
    core = HostCore(num_blocks=64, block_size=4, max_seq_len=64, max_num_seqs=16, max_batched_tokens=64)
    core.sched_add(1, [5, 6, 7], 4)
    core.sched_add(2, [8, 9], 4)
    core.schedule_summary()
    core.update_sampled([40, 41])
    core.sched_add(3, list(range(10, 21)), 4)          # two requests decode, a prompt of 11 tokens arrives
    n, prefill, decode, sampling, shaped = core.schedule_summary()
    assert (n, prefill, decode, sampling, shaped) == (3, 11, 2, 3, False)
    assert (core.plan_rows, core.plan_leading, core.plan_max_run, core.plan_max_context) == (13, 2, 11, 11)
    out = np.full(4096, 77, dtype=np.int32)
    L = core.build_batch_from_plan(out, pad_rows=4 + 64, pad_seqs=4 + 2, pad_logit_rows=6, table_stride=16, pad_leading=4)
    assert (L.rows, L.seqs, L.rows_padded, L.seqs_padded, L.logit_rows, L.logit_rows_padded) == (15, 5, 68, 6, 3, 6)
    run = out[L.run_start:L.run_start + 7].tolist()
    assert run == [0, 1, 2, 3, 4, 15, 15]               # two real single rows, two padding ones, the prompt, a padding sequence
    ctx = out[L.context_lens:L.context_lens + 68]
    assert ctx[:4].tolist() == [4, 3, 0, 0] and ctx[4:15].tolist() == list(range(1, 12)) and not ctx[15:].any()
    slots = out[L.slots[0]:L.slots[0] + 68]
    assert (slots[[0, 1]] >= 0).all() and (slots[[2, 3]] == -1).all() and (slots[4:15] >= 0).all() and (slots[15:] == -1).all()
    assert out[L.row_seq:L.row_seq + 15].tolist() == [0, 1, 2, 3] + [4] * 11
    assert out[L.logit_row_index:L.logit_row_index + 6].tolist() == [0, 1, 14, 0, 0, 0]     # the prompt's last row follows the padding
    tables = out[L.tables[0]:L.tables[0] + 6 * 16].reshape(6, 16)
    assert not tables[2:4].any() and tables[4, :3].tolist() == core.seq_table(3)
    assert out[L.state_slots:L.state_slots + 6].tolist()[2:4] == [-1, -1]
    # without the option nothing changes
    L0 = core.build_batch_from_plan(out)
    assert (L0.rows, L0.seqs) == (13, 3) and out[L0.run_start:L0.run_start + 4].tolist() == [0, 1, 2, 13]
