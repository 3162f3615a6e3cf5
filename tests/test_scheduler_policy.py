"""The scheduling policy (compose / admit / prefix tree / finish / emit).

Three layers:
  * the reference's own test scenarios, replayed on BOTH the product (C++
    scheduler behind the C ABI) and the Python oracle - every expected value
    comes from the reference's tests (cited per test);
  * the reference's unit tests of the prefix tree and detokenizer on the
    product's C++ classes (tests/cpp/policy_unit.cpp) and on the oracle's;
  * a seeded differential run: random request mixes, cancellations and option
    sets through both implementations, compared step by step.

No GPU: the backend is the in-memory FakeBackend of both implementations.
"""

import random
import subprocess
import sys
from pathlib import Path

import pytest

from oracle import scheduler as O
from tests.sched_harness import CONTINUOUS, LOCKSTEP, Harness, pieces

ROOT = Path(__file__).resolve().parent.parent
KINDS = ["product", "oracle"]


def tokens_of(events, index=0):
    return [e[2] for e in events if e[0] == "T" and e[1] == index]


def end_of(events, index=0):
    for e in events:
        if e[0] == "E" and e[1] == index:
            return e[2]
    return None


def ends(events):
    return [e for e in events if e[0] == "E"]


def unit_scheduler(kind, n_batch, mode=CONTINUOUS, **kw):
    """`scheduler(n_batch)` of scheduler.rs:2001-2017."""
    opts = dict(mode=mode, n_batch=n_batch, slow_client_timeout=0.0, prefix_cache=False, event_capacity=256)
    opts.update(kw)
    return Harness(kind, 4, 32, 128, piece_table=["x"] * 100, **opts)


def drain(h):
    """scheduler.rs:2028-2038"""
    for _ in range(200):
        if h.queued() == 0 and h.live() == 0:
            assert h.log()["cells_used"] == 0
            return
        h.pump()
    raise AssertionError("scheduler did not finish")


def finished(h, stream, n_tokens):
    events = h.events(stream)
    assert len(tokens_of(events)) == n_tokens, events
    assert end_of(events) == "MaxTokens", events
    assert h.closed(stream)


# --------------------------------------------------------------------------- scheduler.rs unit tests

@pytest.mark.parametrize("kind", KINDS)
def test_partial_step_failure_keeps_capacity_typed_and_clears_kv_before_reuse(kind):
    # scheduler.rs:2123-2156
    h = Harness(kind, 1, 32, 3, piece_table=["x"] * 100, event_capacity=256)
    h.set("fail_after_steps", 0)
    stream = h.submit([1, 2], [(1, 1)])
    with pytest.raises(h.error_type) as err:
        h.pump()
    assert (err.value.kind, err.value.needed, err.value.available) == ("KvFull", 2, 1)
    assert h.log()["cells_used"] == 0
    events = h.events(stream)
    assert [e[:2] for e in events] == [("X", "KvFull")] and h.closed(stream)
    stream = h.submit([1, 2], [(2, 1)])
    h.pump()
    finished(h, stream, 1)
    assert h.log()["cells_used"] == 0


@pytest.mark.parametrize("kind", KINDS)
def test_a_finished_member_closes_its_stream_and_returns_its_slot_before_its_group_ends(kind):
    # scheduler.rs:2159-2193
    h = unit_scheduler(kind, 8, mode=LOCKSTEP)
    short = h.submit([1, 2], [(1, 1)])
    long = h.submit([1, 2], [(2, 6)])
    h.pump()     # shared prefix
    h.pump()     # both terminal tokens
    finished(h, short, 1)
    h.set_mode(CONTINUOUS)
    nxt = h.submit([3], [(3, 1)] * 3)
    h.pump()
    assert h.queued() == 0, "all three returned/free slots can be reused"
    drain(h)
    finished(h, long, 6)
    assert len(ends(h.events(nxt))) == 3


@pytest.mark.parametrize("kind", KINDS)
def test_cancelling_the_prefill_leader_preserves_the_shared_prefix(kind):
    # scheduler.rs:2196-2211
    h = unit_scheduler(kind, 1, mode=LOCKSTEP)
    first = h.submit([1, 2, 3, 4], [(1, 3)])
    second = h.submit([1, 2, 3, 4], [(2, 3)])
    h.pump()
    h.drop(first)
    drain(h)
    finished(h, second, 3)


@pytest.mark.parametrize("kind", KINDS)
def test_cancelling_an_unsampled_terminal_member_never_decodes_its_returned_slot(kind):
    # scheduler.rs:2214-2231
    h = unit_scheduler(kind, 1, mode=LOCKSTEP)
    first = h.submit([1, 2], [(1, 3)])
    second = h.submit([1, 2], [(2, 3)])
    h.pump()
    h.pump()
    h.drop(second)
    drain(h)
    finished(h, first, 3)
    assert len(h.log()["request_order"]) == 1


@pytest.mark.parametrize("kind", KINDS)
def test_single_token_prompts_and_more_members_than_batch_tokens_make_progress(kind):
    # scheduler.rs:2234-2258
    h = unit_scheduler(kind, 1)
    stream = h.submit([1], [(1, 3)] * 3)
    drain(h)
    events = h.events(stream)
    assert sum(1 for e in events if e[0] == "T") == 9
    assert len(ends(events)) == 3
    assert h.log()["copies"] == [], "there is no shared prefix to copy"


@pytest.mark.parametrize("kind", KINDS)
def test_prefills_progress_while_a_decode_uses_the_entire_batch(kind):
    # scheduler.rs:2261-2282
    h = unit_scheduler(kind, 1)
    first = h.submit([1], [(1, 20)])
    h.pump()
    second = h.submit([2, 3], [(2, 2)])
    for _ in range(8):
        h.pump()
    finished(h, second, 2)
    assert h.live() > 0
    drain(h)
    finished(h, first, 20)


@pytest.mark.parametrize("kind", KINDS)
def test_smaller_arrivals_cannot_overtake_a_request_waiting_for_multiple_slots(kind):
    # scheduler.rs:2285-2313
    h = unit_scheduler(kind, 4)
    first = h.submit([1], [(1, 8)])
    h.pump()
    large = h.submit([2], [(2, 2)] * 4)
    small = h.submit([3], [(3, 1)])
    h.pump()
    assert h.queued() == 2, "the smaller arrival waits its turn"
    drain(h)
    finished(h, first, 8)
    assert len(ends(h.events(large))) == 4
    finished(h, small, 1)


@pytest.mark.parametrize("kind", KINDS)
def test_a_cancelled_queued_request_never_reaches_the_backend(kind):
    # scheduler.rs:2316-2326
    h = unit_scheduler(kind, 4)
    stream = h.submit([1], [(1, 3)])
    h.drop(stream)
    h.pump()
    assert h.log()["steps"] == []


# --------------------------------------------------------------------------- tests/fake_backend.rs

def actor_options(mode, n_batch, **kw):
    """tests/fake_backend.rs:40-52"""
    opts = dict(mode=mode, n_batch=n_batch, queue_capacity=16, event_capacity=256, slow_client_timeout=0.15)
    opts.update(kw)
    return opts


@pytest.mark.parametrize("kind", KINDS)
def test_no_request_starves_and_the_step_budget_is_respected(kind):
    # tests/fake_backend.rs:121-157
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 4))
    streams = [h.submit([10, 11, 12], [(seed, 3)]) for seed in range(1, 7)]
    h.run_until_idle()
    for s in streams:
        events = h.events(s)
        assert len(tokens_of(events)) == 3 and end_of(events) == "MaxTokens", events
    log = h.log()
    assert log["steps"]
    for step in log["steps"]:
        assert sum(n for _, n, _ in step) <= 4, step
    assert log["cells_used"] == 0
    assert len(log["removed"]) >= 6


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("mode,expect_mixed", [(LOCKSTEP, False), (CONTINUOUS, True)])
def test_lockstep_runs_waves_and_continuous_refills_freed_slots(kind, mode, expect_mixed):
    # tests/fake_backend.rs:160-199
    h = Harness(kind, 2, 32, 64, **actor_options(mode, 8))
    streams = [h.submit(p, [(7, b)]) for p, b in zip([[1, 1, 1], [2, 2, 2], [3, 3, 3]], [2, 5, 1])]
    h.run_until_idle()
    for s in streams:
        assert end_of(h.events(s)) is not None
    log = h.log()
    order = log["request_order"]
    assert len(order) == 3
    wave_one, late = order[:2], order[2]
    mixed = any(late in [r for _, _, r in step if r is not None]
                and any(r in wave_one for _, _, r in step if r is not None) for step in log["steps"])
    assert mixed == expect_mixed, log["steps"]


@pytest.mark.parametrize("kind", KINDS)
def test_lockstep_merges_identical_prompts_into_one_prefill_and_copies(kind):
    # tests/fake_backend.rs:202-252
    h = Harness(kind, 4, 32, 128, **actor_options(LOCKSTEP, 8))
    a = h.submit([5, 6, 7, 8], [(1, 2)])
    b = h.submit([5, 6, 7, 8], [(2, 2)])
    h.run_until_idle()
    for s in (a, b):
        events = h.events(s)
        assert len(tokens_of(events)) == 2 and end_of(events) == "MaxTokens"
    log = h.log()
    assert len(log["copies"]) == 1, log["copies"]
    prefix_rows = sum(1 for step in log["steps"] for slot, n, r in step if n == 3 and r is None and slot == 0)
    assert prefix_rows == 1, log["steps"]


@pytest.mark.parametrize("kind", KINDS)
def test_n_greater_than_one_prefills_once_then_copies_to_each_member(kind):
    # tests/fake_backend.rs:255-305
    h = Harness(kind, 4, 32, 128, **actor_options(CONTINUOUS, 8))
    s = h.submit([5, 6, 7, 8, 9], [(1, 2), (2, 2), (3, 2)])
    h.run_until_idle()
    events = h.events(s)
    for index in range(3):
        assert len(tokens_of(events, index)) == 2 and end_of(events, index) == "MaxTokens"
    log = h.log()
    assert len(log["copies"]) == 2 and log["copies"][0][0] == log["copies"][1][0]
    assert sum(1 for step in log["steps"] for _, n, r in step if n == 4 and r is None) == 1
    assert any(sum(1 for _, _, r in step if r is not None) == 3 for step in log["steps"])


@pytest.mark.parametrize("kind", KINDS)
def test_a_cancelled_request_frees_its_slot_at_the_next_step(kind):
    # tests/fake_backend.rs:308-343
    h = Harness(kind, 1, 64, 64, **actor_options(CONTINUOUS, 8))
    long = h.submit([1, 2, 3], [(1, 50)])
    h.pump()
    assert h.events(long)[0][0] == "T"
    h.drop(long)
    second = h.submit([4, 5, 6], [(2, 2)])
    h.run_until_idle()
    events = h.events(second)
    assert len(tokens_of(events)) == 2 and end_of(events) == "MaxTokens"
    log = h.log()
    assert 0 in log["removed"] and log["cells_used"] == 0


@pytest.mark.parametrize("kind", KINDS)
def test_a_full_queue_is_refused_with_a_capacity_error(kind):
    # tests/fake_backend.rs:346-367
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 8, queue_capacity=1))
    first = h.submit([1, 2, 3], [(1, 3)])
    with pytest.raises(h.error_type) as err:
        h.submit([7, 7, 7], [(2, 2)])
    assert err.value.kind == "QueueFull" and err.value.capacity == 1
    h.run_until_idle()
    assert end_of(h.events(first)) == "MaxTokens"


@pytest.mark.parametrize("kind", KINDS)
def test_a_slow_client_is_cancelled_after_the_bounded_backpressure(kind):
    # tests/fake_backend.rs:370-411: a stream nobody drains fills up and is cancelled
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 8, event_capacity=2, slow_client_timeout=0.02))
    slow = h.submit([1, 2, 3], [(1, 30)])        # capacity max(2, 1 + 2) = 3
    quick = h.submit([4, 5, 6], [(2, 2)])
    for _ in range(3):
        h.pump()
    quick_events = h.events(quick)
    assert end_of(quick_events) == "MaxTokens", quick_events
    h.run_until_idle()
    tail = h.events(slow)
    assert all(e[0] == "T" for e in tail) and len(tail) == 3, tail
    assert h.closed(slow)
    assert h.log()["cells_used"] == 0


@pytest.mark.parametrize("kind", KINDS)
def test_an_impossible_reservation_is_refused_instead_of_waiting(kind):
    # tests/fake_backend.rs:452-491
    h = Harness(kind, 2, 32, 10, **actor_options(CONTINUOUS, 8))
    too_big = h.submit([1, 2, 3, 4, 5], [(1, 10)])
    h.run_until_idle()
    events = h.events(too_big)
    assert events[-1][:2] == ("X", "InvalidArgument"), events
    assert events[-1][2] == "the reservation (prompt + max_new_tokens = 15 cells) exceeds the KV pool of 10 cells"
    no_room = h.submit([1] * 32, [(2, 1)])
    h.run_until_idle()
    events = h.events(no_room)
    assert events[-1][:2] == ("X", "InvalidArgument")
    assert events[-1][2] == ("the prompt (32 tokens) leaves no room to generate in the per-sequence context (32)")


@pytest.mark.parametrize("kind", KINDS)
def test_stop_strings_eog_and_budgets_end_the_stream_with_the_right_reason(kind):
    # tests/fake_backend.rs:494-546
    table = pieces(100)
    table[10], table[11], table[12] = "hello", "</end>", "!"
    h = Harness(kind, 2, 32, 64, piece_table=table, **actor_options(CONTINUOUS, 8))
    h.script([10, 11, 12])
    s = h.submit([1, 2, 3], [(1, 10)], stop=["</end>"])
    h.run_until_idle()
    events = h.events(s)
    assert [e[3] for e in events if e[0] == "T"] == ["hello", ""]
    assert end_of(events) == "Stop"
    s = h.submit([1, 2, 3], [(2, 2)])
    h.run_until_idle()
    events = h.events(s)
    assert "".join(e[3] for e in events if e[0] in ("T", "E")) == "hello</end>"
    assert end_of(events) == "MaxTokens"


@pytest.mark.parametrize("kind", KINDS)
def test_eog_ends_the_stream_and_keeps_the_token(kind):
    # tests/fake_backend.rs:549-571
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 8))
    h.set("eog_after", 2)
    s = h.submit([1, 2, 3], [(1, 10)])
    h.run_until_idle()
    events = h.events(s)
    toks = tokens_of(events)
    assert len(toks) == 3 and toks[2] == 99
    assert end_of(events) == "Eog"


@pytest.mark.parametrize("kind", KINDS)
def test_top_logprobs_ride_along_when_requested(kind):
    # tests/fake_backend.rs:574-595
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 8))
    s = h.submit([1, 2, 3], [(1, 2)], n_top_logprobs=3)
    h.run_until_idle()
    toks = [e for e in h.events(s) if e[0] == "T"]
    assert len(toks) == 2
    for t in toks:
        assert len(t[8]) == 3 and t[8][0][0] == 0
        assert t[6] == -0.7          # want_logprob follows n_top_logprobs > 0 (scheduler.rs:1586)


@pytest.mark.parametrize("kind", KINDS)
def test_queued_requests_are_refused_when_the_queue_is_failed(kind):
    # the refusal the actor applies at shutdown (scheduler.rs:631-635, tests/fake_backend.rs:626-652)
    h = Harness(kind, 2, 32, 64, **actor_options(CONTINUOUS, 8))
    streams = [h.submit([1], [(seed, 1)]) for seed in range(1, 4)]
    h.s.fail_queued()
    for s in streams:
        events = h.events(s)
        assert [e[:2] for e in events] == [("X", "Cancelled")]
    assert h.log()["steps"] == []


@pytest.mark.parametrize("kind", KINDS)
def test_invalid_logit_bias_is_refused_without_failing_other_requests(kind):
    # tests/fake_backend.rs:655-686
    h = Harness(kind, 2, 32, 64, **actor_options(LOCKSTEP, 8))
    refused = h.submit([1, 2], [dict(seed=1, max_new_tokens=3, logit_bias=[(100, 1.0)])])
    valid = h.submit([3, 4], [(2, 3)])
    h.run_until_idle()
    assert h.events(refused)[-1][:3] == ("X", "InvalidArgument", "logit_bias token ids must be in 0..100")
    assert end_of(h.events(valid)) == "MaxTokens"


# --------------------------------------------------------------------------- tests/prefix_cache.rs

PROMPT = [1, 2, 3, 4, 5, 6, 7, 8]
SCRIPT = [91, 92]


def cache_harness(kind, n_slots=4, cells=256, **kw):
    """tests/prefix_cache.rs:38-58"""
    opts = dict(mode=CONTINUOUS, n_batch=64, queue_capacity=16, event_capacity=256, slow_client_timeout=0.2,
                prefix_cache=True, min_prefix_len=1)
    fake_kw = {k: kw.pop(k) for k in ("kv_unified", "recurrent") if k in kw}
    opts.update(kw)
    h = Harness(kind, n_slots, 64, cells, **opts)
    h.script(SCRIPT)
    for k, v in fake_kw.items():
        h.set(k, v)
    return h


def run_request(h, prompt, seed, max_new, **kw):
    s = h.submit(prompt, [(seed, max_new)], **kw)
    h.run_until_idle()
    return h.events(s)


def steps_after(h, mark):
    return [(slot, n) for step in h.log()["steps"][mark:] for slot, n, _ in step]


@pytest.mark.parametrize("kind", KINDS)
def test_shared_prefix_is_copied_not_prefilled_and_tokens_are_unchanged(kind):
    # tests/prefix_cache.rs:138-216
    h = cache_harness(kind)
    first = run_request(h, PROMPT, 1, 2)
    assert tokens_of(first) == SCRIPT and end_of(first) == "MaxTokens"
    st = h.kv_stats()
    assert (st["nodes"], st["resident_slots"], st["misses"], st["hits"]) == (1, 1, 1, 0)
    mark = len(h.log()["steps"])
    second = run_request(h, PROMPT + [9, 10], 2, 2)
    assert tokens_of(second) == SCRIPT
    assert any(p0 == 0 and p1 == 8 and src != dst for src, dst, p0, p1 in h.log()["copies"])
    assert sum(n for _, n in steps_after(h, mark)) == 3
    st = h.kv_stats()
    assert (st["hits"], st["prompt_cells"], st["prefilled_cells"]) == (1, 8 + 10, 8 + 2)
    h.pin_prefix(PROMPT + [SCRIPT[0]])
    for i, seed in enumerate(range(3, 6)):
        events = run_request(h, PROMPT + [9 + i], seed, 2)
        assert tokens_of(events) == SCRIPT
    st = h.kv_stats()
    assert st["hits"] == 4
    assert (st["prefilled_cells"] - 8) * 5 < (st["prompt_cells"] - 8)


@pytest.mark.parametrize("kind", KINDS)
def test_fully_cached_prompt_prefills_only_the_last_token(kind):
    # tests/prefix_cache.rs:219-246
    h = cache_harness(kind)
    run_request(h, PROMPT, 1, 2)
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT, 2, 2)
    assert tokens_of(events) == SCRIPT
    rows = steps_after(h, mark)
    assert all(n == 1 for _, n in rows) and len(rows) == 2, rows
    assert any(p0 == 0 and p1 == 7 for _, _, p0, p1 in h.log()["copies"])


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("unified", [True, False])
def test_exact_boundary_hit_uses_a_whole_slot_copy_even_on_a_partitioned_pool(kind, unified):
    # tests/prefix_cache.rs:249-289
    h = cache_harness(kind, kv_unified=unified)
    run_request(h, PROMPT, 1, 2)
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT + SCRIPT, 2, 2)
    assert tokens_of(events) == SCRIPT
    assert any(p0 == -1 and p1 == -1 for _, _, p0, p1 in h.log()["copies"])
    assert all(n == 1 for _, n in steps_after(h, mark))
    assert h.kv_stats()["hits"] == 1


@pytest.mark.parametrize("kind", KINDS)
def test_partitioned_pool_refuses_mid_sequence_hits_and_recomputes(kind):
    # tests/prefix_cache.rs:292-316
    h = cache_harness(kind, kv_unified=False)
    run_request(h, PROMPT, 1, 2)
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT[:6], 2, 1)
    assert tokens_of(events) == [91]
    assert steps_after(h, mark)[0][1] == 6
    st = h.kv_stats()
    assert (st["hits"], st["misses"]) == (0, 2)


@pytest.mark.parametrize("kind", KINDS)
def test_recurrent_models_only_reuse_strict_prefix_boundaries(kind):
    # tests/prefix_cache.rs:319-361
    h = cache_harness(kind, recurrent=True)
    run_request(h, PROMPT, 1, 2)
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT, 2, 1)
    assert tokens_of(events) == [91]
    assert steps_after(h, mark)[0][1] == 8
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT + SCRIPT + [7, 8], 3, 1)
    assert tokens_of(events) == [91]
    assert any(p0 == -1 and p1 == -1 for _, _, p0, p1 in h.log()["copies"])
    assert steps_after(h, mark)[0][1] == 3
    assert h.kv_stats()["hits"] == 1


@pytest.mark.parametrize("kind", KINDS)
def test_lru_eviction_frees_slots_and_pin_protects_a_node(kind):
    # tests/prefix_cache.rs:364-401
    h = cache_harness(kind, swap_min_tokens=(1 << 63))
    run_request(h, PROMPT, 1, 1)
    pin = h.pin_prefix(PROMPT)
    base = len(h.log()["removed"])
    for seed in range(2, 6):
        run_request(h, [50 + seed, 60], seed, 1)
    assert h.kv_stats()["evictions"] >= 1
    assert 0 not in h.log()["removed"][base:]
    assert h.unpin(pin)
    run_request(h, [70, 71], 9, 1)
    assert 0 in h.log()["removed"][base:]


@pytest.mark.parametrize("kind", KINDS)
def test_long_nodes_swap_to_a_host_snapshot_and_restore_on_a_later_hit(kind):
    # tests/prefix_cache.rs:404-452
    h = cache_harness(kind, swap_min_tokens=1, max_snapshot_bytes=1 << 20)
    run_request(h, PROMPT, 1, 2)
    for seed in range(2, 6):
        run_request(h, [50 + seed, 60], seed, 1)
    assert any(flags == 0 and n > 0 for _, flags, n in h.log()["saves"])
    st = h.kv_stats()
    assert st["swaps"] >= 1 and st["snapshot_bytes"] > 0
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT + [SCRIPT[0], 9], 6, 2)
    assert tokens_of(events) == SCRIPT
    assert any(flags == 0 and n > 0 for _, flags, n in h.log()["loads"])
    assert sum(n for _, n in steps_after(h, mark)) == 2


@pytest.mark.parametrize("kind", KINDS)
def test_a_weights_version_change_drops_the_tree_and_the_next_request_is_cold(kind):
    # tests/prefix_cache.rs:455-484
    h = cache_harness(kind)
    run_request(h, PROMPT, 1, 2)
    assert h.kv_stats()["nodes"] == 1
    h.set("bump_weights_version")
    mark = len(h.log()["steps"])
    events = run_request(h, PROMPT + [9], 2, 1)
    assert tokens_of(events) == [91]
    assert steps_after(h, mark)[0][1] == 9
    assert h.log()["removed"]
    st = h.kv_stats()
    assert (st["misses"], st["hits"]) == (2, 0)


@pytest.mark.parametrize("kind", KINDS)
def test_a_hit_charges_only_the_suffix_against_the_cell_budget(kind):
    # tests/prefix_cache.rs:487-511
    h = cache_harness(kind, cells=19)
    run_request(h, PROMPT, 1, 2)
    events = run_request(h, PROMPT + [9], 2, 2)
    assert end_of(events) == "MaxTokens" and tokens_of(events) == SCRIPT
    assert h.kv_stats()["hits"] == 1


@pytest.mark.parametrize("kind", KINDS)
def test_a_retained_turn_survives_slot_pressure_until_its_continuation_releases_it(kind):
    # tests/prefix_cache.rs:514-566
    h = cache_harness(kind, swap_min_tokens=(1 << 63))
    first = run_request(h, PROMPT, 1, 1, retention=("a", None))
    assert ends(first)[0][4] == 0, "a cold prompt reuses nothing"
    base = len(h.log()["removed"])
    for seed in range(2, 6):
        run_request(h, [50 + seed, 60], seed, 1)
    assert 0 not in h.log()["removed"][base:]
    second = run_request(h, PROMPT + [9, 10], 6, 1, retention=("b", "a"))
    assert tokens_of(second) == [SCRIPT[0]]
    assert ends(second)[0][4] == len(PROMPT)
    for seed in range(7, 11):
        run_request(h, [50 + seed, 61], seed, 1)
    assert 0 in h.log()["removed"][base:]


@pytest.mark.parametrize("kind", KINDS)
def test_a_retention_gives_way_to_an_admission_that_needs_its_slot(kind):
    # tests/prefix_cache.rs:569-591
    h = cache_harness(kind)
    run_request(h, PROMPT, 1, 1, retention=("a", None))
    s = h.submit([80, 81], [(seed, 1) for seed in range(1, 5)])
    h.run_until_idle()
    assert len(ends(h.events(s))) == 4
    assert 0 in h.log()["removed"]


@pytest.mark.parametrize("kind", KINDS)
def test_an_expired_retention_is_released_at_the_next_admission(kind):
    # tests/prefix_cache.rs:594-615
    h = cache_harness(kind, swap_min_tokens=(1 << 63), retain_ttl=0.0)
    run_request(h, PROMPT, 1, 1, retention=("a", None))
    base = len(h.log()["removed"])
    for seed in range(2, 6):
        run_request(h, [50 + seed, 60], seed, 1)
    assert 0 in h.log()["removed"][base:]


# --------------------------------------------------------------------------- tests/adapters.rs, tests/row_adapters.rs

def adapter_harness(kind, n_slots=2, cells=64, row_adapters=False, table=None, mode=CONTINUOUS):
    """tests/adapters.rs:36-55, tests/row_adapters.rs:29-46"""
    h = Harness(kind, n_slots, 32, cells, piece_table=table, mode=mode, n_batch=16, queue_capacity=16,
                event_capacity=64, slow_client_timeout=0.0)
    if row_adapters:
        h.set("row_adapters", 1)
    return h


def run_all(h, requests):
    streams = [h.submit(prompt, [(seed, max_new)], adapter=adapter) for prompt, seed, max_new, adapter in requests]
    h.run_until_idle()
    return [h.events(s) for s in streams]


def has_error(events):
    return any(e[0] == "X" for e in events)


@pytest.mark.parametrize("kind", KINDS)
def test_same_adapter_requests_batch_and_never_reactivate(kind):
    # tests/adapters.rs:73-92; the fake registers the adapter directly (backend_mut().load_adapter)
    h = adapter_harness(kind)
    h.register_adapter("a")
    out = run_all(h, [([1, 2, 3], 1, 3, "a"), ([1, 2, 3], 2, 3, "a")])
    assert not any(has_error(e) for e in out)
    assert sum(1 for op, _ in h.log()["adapter_ops"] if op == "activate") == 1


@pytest.mark.parametrize("kind", KINDS)
def test_adapters_serialize_one_at_a_time_and_each_switch_invalidates_the_kv(kind):
    # tests/adapters.rs:95-131 (prompts of 8 tokens so the finished sequence becomes a tree node)
    h = adapter_harness(kind)
    h.register_adapter("a")
    h.register_adapter("b")
    out = run_all(h, [(PROMPT, 1, 3, "a")])
    assert not has_error(out[0]) and h.kv_stats()["resident_slots"] > 0
    out = run_all(h, [(PROMPT, 2, 3, "b")])
    assert not has_error(out[0])
    assert ("activate", "b") in h.log()["adapter_ops"]
    st = h.kv_stats()
    assert st["nodes"] == 1 and st["misses"] == 2


@pytest.mark.parametrize("kind", KINDS)
def test_a_step_never_mixes_adapters_even_with_free_slots(kind):
    # tests/adapters.rs:134-158
    h = adapter_harness(kind)
    h.register_adapter("a")
    h.register_adapter("b")
    first = h.submit([1, 2, 3], [(1, 3)], adapter="a")
    second = h.submit([1, 2, 3], [(2, 3)], adapter="b")
    seen = []
    while not (h.queued() == 0 and h.live() == 0):
        h.pump()
        acts = [name for op, name in h.log()["adapter_ops"] if op == "activate"]
        seen.append(acts[-1] if acts else None)
    assert ends(h.events(first)) and ends(h.events(second))
    assert sum(1 for a, b in zip(seen, seen[1:]) if a != b) <= 1
    assert "a" in seen and "b" in seen


@pytest.mark.parametrize("kind", KINDS)
def test_a_request_for_an_unregistered_adapter_is_refused_not_hung(kind):
    # tests/adapters.rs:161-183
    h = adapter_harness(kind)
    s = h.submit([1, 2, 3], [(1, 3)], adapter="ghost")
    h.run_until_idle()
    events = h.events(s)
    assert events and events[-1][0] == "X" and "no adapter registered" in events[-1][2]


ROW_PROMPT = [1, 2, 3, 4, 5, 6, 7, 8]


@pytest.mark.parametrize("kind", KINDS)
def test_per_row_adapters_and_the_base_model_share_steps(kind):
    # tests/row_adapters.rs:74-110
    h = adapter_harness(kind, 4, 128, row_adapters=True)
    h.load_adapter("a")
    h.load_adapter("b")
    out = run_all(h, [(ROW_PROMPT, 1, 4, "a"), (ROW_PROMPT, 2, 4, "b"), (ROW_PROMPT, 3, 4, None)])
    assert not any(has_error(e) for e in out)
    log = h.log()
    assert not any(op == "activate" for op, _ in log["adapter_ops"])
    assert any(1 in rows and 2 in rows and 0 in rows for rows in log["step_adapters"])


@pytest.mark.parametrize("kind", KINDS)
def test_a_prefix_is_reused_under_its_own_adapter_only(kind):
    # tests/row_adapters.rs:113-127
    h = adapter_harness(kind, 4, 128, row_adapters=True)
    h.load_adapter("a")
    h.load_adapter("b")
    for adapter in ("a", "b"):
        assert not has_error(run_all(h, [(ROW_PROMPT, 1, 2, adapter)])[0])
    st = h.kv_stats()
    assert (st["hits"], st["misses"]) == (0, 2)
    assert not has_error(run_all(h, [(ROW_PROMPT, 3, 2, "a")])[0])
    assert h.kv_stats()["hits"] == 1


@pytest.mark.parametrize("kind", KINDS)
def test_a_reloaded_adapter_keeps_live_requests_on_the_old_generation(kind):
    # tests/row_adapters.rs:130-160
    h = adapter_harness(kind, 4, 128, row_adapters=True)
    h.load_adapter("a")
    live = h.submit(ROW_PROMPT, [(1, 6)], adapter="a")
    h.pump()
    assert h.live() == 1
    h.load_adapter("a")
    nxt = h.submit(ROW_PROMPT, [(2, 2)], adapter="a")
    h.run_until_idle()
    assert ends(h.events(live)) and ends(h.events(nxt))
    log = h.log()
    assert ("unload_row", "1") in log["adapter_ops"] and ("unload_row", "2") not in log["adapter_ops"]
    ids = [a for rows in log["step_adapters"] for a in rows]
    assert 1 in ids and 2 in ids


@pytest.mark.parametrize("kind", KINDS)
def test_an_unloaded_adapter_refuses_new_requests_and_frees_its_prefixes(kind):
    # tests/row_adapters.rs:163-187
    h = adapter_harness(kind, 4, 128, row_adapters=True)
    h.load_adapter("a")
    assert not has_error(run_all(h, [(ROW_PROMPT, 1, 2, "a")])[0])
    assert h.kv_stats()["resident_slots"] > 0
    h.unload_adapter("a")
    assert h.kv_stats()["resident_slots"] == 0
    assert ("unload_row", "1") in h.log()["adapter_ops"]
    assert has_error(run_all(h, [(ROW_PROMPT, 2, 2, "a")])[0])
    with pytest.raises(h.error_type):
        h.unload_adapter("a")


@pytest.mark.parametrize("kind", KINDS)
def test_a_backend_without_per_row_support_keeps_serializing(kind):
    # tests/row_adapters.rs:190-219
    h = adapter_harness(kind, 2, 64, table=["x"] * 100)
    h.load_adapter("a")
    assert not has_error(run_all(h, [(ROW_PROMPT, 1, 2, "a")])[0])
    log = h.log()
    assert ("activate", "a") in log["adapter_ops"]
    assert all(a == 0 for rows in log["step_adapters"] for a in rows)


@pytest.mark.parametrize("kind", KINDS)
def test_a_serialized_replacement_retires_the_previous_row_adapter(kind):
    # tests/row_adapters.rs:222-248
    h = adapter_harness(kind, 4, 128, row_adapters=True)
    h.load_adapter("a")
    live = h.submit(ROW_PROMPT, [(1, 6)], adapter="a")
    h.pump()
    h.set("row_adapters", 0)
    h.load_adapter("a")
    nxt = h.submit(ROW_PROMPT, [(2, 2)], adapter="a")
    h.run_until_idle()
    for s in (live, nxt):
        events = h.events(s)
        assert not has_error(events) and ends(events)
    log = h.log()
    assert ("unload_row", "1") in log["adapter_ops"]
    assert [name for op, name in log["adapter_ops"] if op == "activate"][-1] == "a"


@pytest.mark.parametrize("kind", KINDS)
def test_unloading_a_row_adapter_never_reactivates_an_old_named_adapter(kind):
    # tests/row_adapters.rs:251-265
    h = adapter_harness(kind, 4, 128)
    h.load_adapter("a")
    h.set("row_adapters", 1)
    h.load_adapter("a")
    h.unload_adapter("a")
    assert has_error(run_all(h, [(ROW_PROMPT, 1, 2, "a")])[0])
    h.load_adapter("a")
    assert not has_error(run_all(h, [(ROW_PROMPT, 1, 2, "a")])[0])


# --------------------------------------------------------------------------- the oracle's own tree and detokenizer

def test_oracle_prefix_tree_reference_unit_tests():
    # crates/retrograd-infer/src/kv.rs:558-700
    def tree_with(paths):
        t = O.PrefixTree()
        for i, p in enumerate(paths):
            t.insert(0, p, i + 1)
        return t
    yes = lambda n, h: True
    t = tree_with([[1, 2, 3, 4], [1, 2, 9, 9]])
    assert t.longest_prefix(0, [1, 2, 3, 4, 5], True, yes) == (1, 4)
    assert t.longest_prefix(0, [1, 2, 9, 8], True, yes)[1] == 3
    assert t.longest_prefix(0, [1, 2, 9, 8], False, yes)[1] == 2
    t = tree_with([[1, 2, 3, 4]])
    assert t.longest_prefix(0, [1, 2], True, yes) == (1, 2)
    assert t.longest_prefix(0, [1, 2], False, yes) is None
    t = tree_with([[1, 2, 3], [1, 2, 9]])
    with_slots = lambda n, h: t.nodes[n].slot is not None
    assert t.longest_prefix(0, [1, 2, 7], True, with_slots)[1] == 2
    assert t.longest_prefix(0, [1, 2, 7], False, with_slots) is None
    t = tree_with([[1, 2, 3], [1, 2, 3, 4]])
    assert t.longest_prefix(0, [1, 2, 3, 4, 5], False, lambda n, h: n != 2) == (1, 3)

    t = tree_with([[7, 7, 7]])
    node, attached = t.insert(0, [7, 7, 7], 42)
    assert not attached and t.slot(node) == 1
    pin = t.pin_at(0, [7, 7, 7])
    assert t.eviction_candidate() is None
    assert t.unpin(pin) and t.eviction_candidate() == node and not t.unpin(pin)
    assert t.pin_at(0, [8, 8]) is None

    t = tree_with([[1], [1, 2]])
    t.attach_snapshot(2, bytes(100))
    assert t.snapshot_bytes == 100
    assert len(t.clear()) == 2 and t.node_count() == 0 and t.snapshot_bytes == 0

    t = tree_with([[1, 2], [5, 6]])
    node, _ = t.insert(0, [1, 2], 9)
    t.remove(node)
    assert t.node_count() == 1 and t.longest_prefix(0, [1, 2, 3], True, yes) is None
    reused, attached = t.insert(0, [7, 8], 3)
    assert attached and reused == node and t.node_count() == 2

    t = O.PrefixTree()
    t.insert(0, [1, 2, 3, 4], 1)
    t.insert(7, [1, 2, 3, 4], 2)
    t.insert(7, [1, 2, 9], 3)
    base, hit = t.longest_prefix(0, [1, 2, 3, 4, 5], False, yes)
    assert (t.slot(base), hit) == (1, 4)
    routed, hit = t.longest_prefix(7, [1, 2, 3, 4, 5], False, yes)
    assert (t.slot(routed), hit) == (2, 4)
    assert t.longest_prefix(8, [1, 2, 3, 4], True, yes) is None
    assert t.node_count() == 4
    pin = t.pin_at(7, [1, 2, 9])
    assert sorted(t.drop_namespace(7)) == [2, 3]
    assert not t.unpin(pin)
    assert t.longest_prefix(7, [1, 2, 3, 4], True, yes) is None
    assert t.node_count() == 1 and t.resident_slots() == [1]
    t.insert(7, [5, 6], 4)
    assert t.node_count() == 2


def test_oracle_detokenizer_reference_unit_tests():
    # crates/retrograd-infer/src/detok.rs:134-210
    party = "🎉".encode()
    d = O.Detokenizer([])
    assert d.push_bytes(b"ok ") == ("ok ", False)
    assert d.push_bytes(party[:2]) == ("", False)
    assert d.push_bytes(party[2:]) == ("🎉", False)
    d = O.Detokenizer(["STOP"])
    assert d.push_bytes(b"abcST") == ("abc", False)
    assert d.push_bytes(b"OP") == ("", True)
    assert d.push_bytes(b"xyz") == ("", True)
    d = O.Detokenizer(["</end>"])
    assert d.push_bytes(b"answer</end>ignored") == ("answer", True)
    d = O.Detokenizer(["STOP"])
    assert d.push_bytes(b"abST")[0] == "ab" and d.finish() == "ST"
    d = O.Detokenizer(["abc"])
    emitted = ""
    for piece in "xabde":
        text, stopped = d.push_bytes(piece.encode())
        assert not stopped
        emitted += text
    assert emitted + d.finish() == "xabde"
    for chunks in ([b"\xffvalid"], [b"\xf0\x9f", b"ok"], [b"ok\xf0\x9f"]):
        d = O.Detokenizer([])
        text = "".join(d.push_bytes(c)[0] for c in chunks) + d.finish()
        assert text == b"".join(chunks).decode("utf-8", "replace")
    d = O.Detokenizer(["abcdef"])
    assert d.push_bytes(b"zzabc") == ("zz", False)
    assert d.push_bytes(b"x") == ("abcx", False)


def test_product_prefix_tree_and_detokenizer_reference_unit_tests(tmp_path):
    exe = tmp_path / "policy_unit"
    subprocess.run(["g++", "-std=c++17", "-O1", "-o", str(exe), str(ROOT / "tests/cpp/policy_unit.cpp"),
                    str(ROOT / "retrograd_amd/csrc/sched/prefix_tree.cpp")], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


# --------------------------------------------------------------------------- product vs oracle, step by step

def _random_piece_table(rng):
    table = pieces(100)
    for t, text in ((10, "hello"), (11, "</end>"), (12, "!"), (13, "STOP"), (14, "ST"), (15, "OP"), (16, "é")):
        table[t] = text
    table[17], table[18] = "🎉".encode()[:2], "🎉".encode()[2:]
    table[19] = b"\xff"
    return table


@pytest.mark.parametrize("seed", range(24))
def test_product_matches_the_oracle_on_random_workloads(seed):
    rng = random.Random(1000 + seed)
    n_slots = rng.choice([1, 2, 4, 6])
    n_ctx = rng.choice([24, 48])
    cells = rng.choice([n_ctx, 2 * n_ctx, n_slots * n_ctx])
    opts = dict(mode=rng.choice([LOCKSTEP, CONTINUOUS]), n_batch=rng.choice([1, 2, 5, 16]), queue_capacity=8,
                event_capacity=rng.choice([4, 64]), slow_client_timeout=0.0, prefix_cache=rng.random() < 0.8,
                min_prefix_len=rng.choice([1, 4]), swap_min_tokens=rng.choice([1, 6, 1 << 63]),
                max_snapshot_bytes=rng.choice([16, 48, 1 << 20]), max_retained=rng.choice([0, 1, 8]),
                retain_ttl=300.0)
    table = _random_piece_table(rng)
    hs = [Harness(kind, n_slots, n_ctx, cells, piece_table=table, **opts) for kind in KINDS]
    script = [rng.choice([10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 3, 4]) for _ in range(rng.randint(1, 6))]
    use_script = rng.random() < 0.7
    unified, recurrent = rng.random() < 0.8, rng.random() < 0.15
    eog_after = rng.choice([-1, -1, 2, 5])
    for h in hs:
        if use_script:
            h.script(script)
        h.set("kv_unified", unified)
        h.set("recurrent", recurrent)
        h.set("eog_after", eog_after)
    row_adapters = rng.random() < 0.5
    for h in hs:
        h.set("row_adapters", row_adapters)
    names = ["a", "b", "ghost"]
    prompts = [[rng.randrange(1, 9) for _ in range(rng.randint(1, 12))] for _ in range(4)]
    streams = [[], []]
    pins = [[], []]

    def same(what, a, b):
        assert a == b, "%s differs (seed %d):\nproduct %r\noracle  %r" % (what, seed, a, b)

    for it in range(rng.randint(20, 60)):
        action = rng.random()
        if action < 0.45:
            base = rng.choice(prompts)
            prompt = base[:rng.randint(1, len(base))] + [rng.randrange(1, 9) for _ in range(rng.randint(0, 3))]
            n = rng.choice([1, 1, 1, 2, 3])
            sampling = [dict(seed=rng.randrange(4), max_new_tokens=rng.randint(1, 7),
                             temperature=rng.choice([1.0, 0.5]), top_k=rng.choice([0, 1])) for _ in range(n)]
            kw = {}
            if rng.random() < 0.4:
                kw["stop"] = rng.sample(["</end>", "STOP", "!", "lo"], rng.randint(1, 2))
            if rng.random() < 0.3:
                kw["n_top_logprobs"] = rng.randint(1, 3)
            if rng.random() < 0.2:
                kw["logprobs"] = True
            if rng.random() < 0.2:
                kw["unparse_special"] = True
            if rng.random() < 0.25:
                kw["retention"] = (rng.choice("ab"), rng.choice([None, "a", "b"]))
            if rng.random() < 0.35:
                kw["adapter"] = rng.choice(names)
            outcome = []
            for i, h in enumerate(hs):
                try:
                    streams[i].append(h.submit(prompt, sampling, **dict(kw)))
                    outcome.append("ok")
                except h.error_type as e:
                    outcome.append(e.kind)
            same("submit outcome", outcome[0], outcome[1])
        elif action < 0.55 and streams[0]:
            k = rng.randrange(len(streams[0]))
            for i, h in enumerate(hs):
                h.drop(streams[i][k])
        elif action < 0.6:
            prefix = rng.choice(prompts)[:rng.randint(1, 6)]
            got = []
            for i, h in enumerate(hs):
                try:
                    pins[i].append(h.pin_prefix(prefix))
                    got.append("ok")
                except h.error_type as e:
                    got.append(e.kind)
            same("pin outcome", got[0], got[1])
        elif action < 0.63 and pins[0]:
            k = rng.randrange(len(pins[0]))
            same("unpin", hs[0].unpin(pins[0][k]), hs[1].unpin(pins[1][k]))
        elif action < 0.66:
            for h in hs:
                h.set("bump_weights_version")
        elif action < 0.72:
            name, unload = rng.choice(names[:2]), rng.random() < 0.3
            got = []
            for h in hs:
                try:
                    h.unload_adapter(name) if unload else h.load_adapter(name)
                    got.append("ok")
                except h.error_type as e:
                    got.append(e.kind)
            same("adapter operation", got[0], got[1])
        elif action < 0.74:
            flip = rng.random() < 0.5
            for h in hs:
                h.set("row_adapters", flip)
        else:
            results = []
            for h in hs:
                try:
                    results.append(h.pump())
                except h.error_type as e:
                    results.append((e.kind, e.needed, e.available))
            same("pump result", results[0], results[1])
        same("queued", hs[0].queued(), hs[1].queued())
        same("live", hs[0].live(), hs[1].live())
        if rng.random() < 0.3:
            for k in range(len(streams[0])):
                same("events of stream %d" % k, hs[0].events(streams[0][k]), hs[1].events(streams[1][k]))
    for h in hs:
        for _ in range(400):
            if h.queued() == 0 and h.live() == 0:
                break
            try:
                h.pump()
            except h.error_type:
                pass
    for k in range(len(streams[0])):
        same("final events of stream %d" % k, hs[0].events(streams[0][k]), hs[1].events(streams[1][k]))
        same("closed %d" % k, hs[0].closed(streams[0][k]), hs[1].closed(streams[1][k]))
    la, lb = hs[0].log(), hs[1].log()
    for key in la:
        same(key, la[key], lb[key])
    same("kv stats", hs[0].kv_stats(), hs[1].kv_stats())


# --------------------------------------------------------------------------- the rollout configuration's plan shape

def _rollout_requests(seed, n_requests=32, common=2048, lo=32, hi=512, vocab=1000):
    rng = random.Random(seed)
    prefix = [rng.randrange(1, vocab - 1) for _ in range(common)]
    return [prefix + [rng.randrange(1, vocab - 1) for _ in range(rng.randint(lo, hi))] for _ in range(n_requests)]


def _rollout_harness(kind, n_slots, n_ctx_seq=4096, vocab=1000, n_batch=512, **kw):
    opts = dict(mode=CONTINUOUS, n_batch=n_batch, queue_capacity=64, event_capacity=4096, slow_client_timeout=0.0,
                prefix_cache=True, min_prefix_len=8, swap_min_tokens=1 << 62)
    opts.update(kw)
    return Harness(kind, n_slots, n_ctx_seq, n_slots * n_ctx_seq, vocab=vocab, eos=vocab - 1,
                   piece_table=["x"] * vocab, **opts)


def test_rollout_shape_with_a_slot_per_member_is_32_cold_prefills_and_224_whole_slot_copies():
    """32 prompts (2048 common tokens + 32..512 of their own), 8 members each, 256 slots, nothing pinned
    (scheduler.rs:1094-1121, 1326-1336, 1816-1843): the prefix tree only learns a path when a member finishes, and
    all 32 groups are admitted in one pass, so every group is a cold miss that prefills its whole prompt but the
    last token once, copies the leader's slot to its 7 members (seq_cp(leader, member, -1, -1)) and reports
    cached_tokens = 0. The product's plan must equal the policy oracle's call for call."""
    prompts = _rollout_requests(5)
    hs = {kind: _rollout_harness(kind, 256) for kind in KINDS}
    events = {}
    for kind, h in hs.items():
        streams = [h.submit(p, [dict(seed=100 * i + m, max_new_tokens=3, temperature=1.0, top_k=40) for m in range(8)])
                   for i, p in enumerate(prompts)]
        h.run_until_idle()
        events[kind] = [h.events(s) for s in streams]
    la, lb = hs["product"].log(), hs["oracle"].log()
    for key in la:
        assert la[key] == lb[key], key
    assert events["product"] == events["oracle"]
    assert hs["product"].kv_stats() == hs["oracle"].kv_stats()
    st = hs["product"].kv_stats()
    total = sum(len(p) for p in prompts)
    assert (st["hits"], st["misses"]) == (0, 32)
    assert st["prompt_cells"] == total
    # the leader prefills len - 1 tokens; the last prompt token is every member's own terminal row and is not counted
    assert st["prefilled_cells"] == total - 32
    copies = la["copies"]
    assert len(copies) == 224 and all(p0 == -1 and p1 == -1 for _, _, p0, p1 in copies)
    leaders = {}
    for src, dst, _, _ in copies:
        leaders.setdefault(src, []).append(dst)
    assert len(leaders) == 32 and all(len(v) == 7 for v in leaders.values())
    assert len({d for v in leaders.values() for d in v} | set(leaders)) == 256        # every slot used exactly once
    for ev in events["product"]:
        e = ends(ev)
        assert len(e) == 8 and all(x[2] == "MaxTokens" and x[4] == 0 for x in e)      # cached_tokens = 0
        assert all(len(tokens_of(ev, m)) == 3 for m in range(8))
    # the common prefix was prefilled once per request: 32 x 2048 tokens and more in prefill rows
    prefill_tokens = sum(n for step in la["steps"] for _, n, r in step if r is None)
    assert prefill_tokens == total - 32


def test_rollout_shape_with_fewer_slots_than_members_reuses_the_common_prefix_by_partial_copies():
    """72 slots for 256 members, the 32 requests arriving in four waves of 8. (Queued all at once they would never hit:
    a waiting group is admitted the moment eight slots can be freed, which evicts exactly the eight dormant nodes
    the tree holds - the policy oracle shows hits = 0 there too.) Groups of the later waves find the common prefix
    in the tree and take a partial copy [0, hit) from the deepest slot-bearing node (kv.rs:246-260,
    scheduler.rs:1446-1522) into their leader, then whole-slot copies to the members; the hit is the 2048 common
    tokens, or one more where two prompts happen to continue alike. Product and policy oracle must agree on every
    step, copy, removal, event and counter."""
    prompts = _rollout_requests(6)
    hs = {kind: _rollout_harness(kind, 72) for kind in KINDS}
    events = {kind: [] for kind in KINDS}
    for kind, h in hs.items():
        for w in range(4):
            streams = [h.submit(p, [dict(seed=100 * i + m, max_new_tokens=2 + (i + m) % 3, temperature=1.0, top_k=40)
                                    for m in range(8)]) for i, p in enumerate(prompts[8 * w:8 * w + 8])]
            h.run_until_idle()
            events[kind] += [h.events(s) for s in streams]
    la, lb = hs["product"].log(), hs["oracle"].log()
    for key in la:
        assert la[key] == lb[key], key
    assert events["product"] == events["oracle"]
    assert hs["product"].kv_stats() == hs["oracle"].kv_stats()
    st = hs["product"].kv_stats()
    assert st["misses"] == 8 and st["hits"] == 24, st            # the first wave is cold, every later group hits
    partial = [(s_, d, p0, p1) for s_, d, p0, p1 in la["copies"] if p0 == 0]
    assert len(partial) == 24 and all(p1 in (2048, 2049) for _, _, _, p1 in partial), partial[:3]
    assert len([c for c in la["copies"] if c[2] == -1 and c[3] == -1]) == 224
    cached = [ends(ev)[0][4] for ev in events["product"]]
    assert cached[:8] == [0] * 8 and sorted(cached[8:]) == sorted(p1 for _, _, _, p1 in partial)
    for ev in events["product"]:
        assert len({x[4] for x in ends(ev)}) == 1                # every member of a group reports its group's hit
    total = sum(len(p) for p in prompts)
    assert st["prefilled_cells"] == total - 32 - sum(cached)
