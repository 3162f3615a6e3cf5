"""The synchronous driver of the scheduler: `run_requests` (submit a batch, pump until every
request has ended, one structured outcome per request) and `lend_slot`, replayed from the
reference's crates/retrograd-infer/tests/sync_driver.rs:52-372 on BOTH implementations - the
product (C++ scheduler behind the C ABI, driver in retrograd_amd/scheduler.py) and the Python
oracle - with the reference's expected values, and the two compared with each other.

No GPU: the backend is the in-memory FakeBackend of both implementations."""
import pytest

from tests.sched_harness import CONTINUOUS, LOCKSTEP, Harness

KINDS = ["product", "oracle"]


def sched(kind, mode, queue_capacity, **kw):
    """`scheduler(fake(), mode, queue_capacity)` of sync_driver.rs:29-49: 4 slots, 32 positions each, 128 cells."""
    opts = dict(mode=mode, n_batch=16, queue_capacity=queue_capacity, event_capacity=8, slow_client_timeout=0.0)
    opts.update(kw)
    return Harness(kind, 4, 32, 128, **opts)


@pytest.mark.parametrize("kind", KINDS)
def test_run_requests_collects_every_completion_in_submission_order(kind):      # sync_driver.rs:52-102
    h = sched(kind, LOCKSTEP, 16)
    outcomes = h.run_requests([([1, 2, 3], [(7, 5)]), ([4, 5], [(1, 4), (2, 4), (3, 4)]), ([9, 8, 7, 6], [(8, 6)])])
    assert [len(c) for c, _ in outcomes] == [1, 3, 1]
    for completions, error in outcomes:
        assert error is None
        for tokens, logprobs, forced, _text, finish in completions:
            assert finish == "MaxTokens" and len(tokens) == len(logprobs) == len(forced) and not any(forced)
    assert [len(c[0][0]) for c, _ in outcomes] == [5, 4, 6]
    streams = [c[0] for c in outcomes[1][0]]
    assert streams[0] != streams[1] and streams[1] != streams[2], "distinct seeds give distinct streams"
    assert h.is_idle()


def test_run_requests_is_identical_on_the_product_and_the_oracle_and_per_seed():   # sync_driver.rs:105-117
    batch = [([1, 2, 3], [(42, 8)]), ([4, 5], [(1, 4), (2, 4)]), ([1, 2, 3, 4, 5, 6, 7, 8, 9], [(3, 6)])]
    runs = [sched(kind, mode, 16).run_requests(batch) for kind in KINDS for mode in (LOCKSTEP, CONTINUOUS) for _ in (0, 1)]
    assert all(r == runs[0] for r in runs[:2]) and runs[0] == runs[4], "same seed, same tokens; product == oracle"
    assert runs[2] == runs[3] == runs[6]


@pytest.mark.parametrize("kind", KINDS)
def test_run_requests_submits_beyond_the_queue_capacity_as_slots_free(kind):    # sync_driver.rs:120-132
    h = sched(kind, CONTINUOUS, 1)
    outcomes = h.run_requests([([1, 2], [(seed, 4)]) for seed in range(3)])
    assert len(outcomes) == 3
    for completions, error in outcomes:
        assert error is None and len(completions[0][0]) == 4


@pytest.mark.parametrize("kind", KINDS)
def test_an_impossible_reservation_comes_back_as_an_outcome_error(kind):        # sync_driver.rs:135-145
    h = sched(kind, LOCKSTEP, 16)
    # the per-sequence context is 32 positions: a 32-token prompt leaves no room to generate
    outcomes = h.run_requests([([7] * 32, [(1, 4)])])
    assert len(outcomes) == 1
    completions, error = outcomes[0]
    assert error is not None, "the refusal is reported"
    assert completions[0][4] is None


@pytest.mark.parametrize("kind", KINDS)
def test_an_eog_token_is_kept_and_ends_the_completion(kind):                    # sync_driver.rs:148-160
    h = sched(kind, LOCKSTEP, 16)
    h.set("eog_after", 3)
    (completions, _), = h.run_requests([([1, 2], [(5, 10)])])
    tokens, _, _, _, finish = completions[0]
    assert finish == "Eog"
    assert len(tokens) == 4 and tokens[3] == 99, "three sampled tokens plus the EOG"


@pytest.mark.parametrize("kind", KINDS)
def test_a_dropped_stream_is_removed_at_the_next_step(kind):                    # sync_driver.rs:163-190
    h = Harness(kind, 4, 32, 128, mode=CONTINUOUS, n_batch=16, slow_client_timeout=0.0, prefix_cache=False)
    stream = h.submit([1, 2, 3], [(1, 8)])
    h.pump()
    assert h.live() == 1
    h.drop(stream)
    h.run_until_idle()
    assert h.is_idle()
    assert h.log()["removed"], "the cancelled sequence's slot was released"


@pytest.mark.parametrize("kind", KINDS)
def test_initialize_clears_residue_left_by_earlier_calls(kind):                 # sync_driver.rs:193-225
    h = Harness(kind, 4, 32, 128, mode=LOCKSTEP, prefix_cache=True, min_prefix_len=1)
    h.run_requests([([1, 2], [(1, 4)])])
    assert h.cells_used() > 0, "a finished sequence stays resident for the prefix cache"
    # a fresh start on the same backend begins from empty slots, like the batched generators
    h.s.initialize()
    assert h.live() == 0 and h.cells_used() == 0


@pytest.mark.parametrize("kind", KINDS)
def test_a_step_failure_is_returned_and_fails_the_live_requests(kind):          # sync_driver.rs:228-314
    h = Harness(kind, 4, 32, 128, mode=LOCKSTEP, slow_client_timeout=0.0)
    h.set("fail_after_steps", 0)                      # every step fails
    stream = h.submit([1, 2], [(1, 4)])
    with pytest.raises(h.error_type) as err:
        h.pump()
    # the reference wraps its fake in a backend whose step returns Failed("boom"); the fakes' own scripted
    # failure (fake.rs fail_after_steps) is a Backend error - either way it is the backend's error that surfaces
    assert err.value.kind in ("Failed", "Backend")
    assert h.is_idle(), "the failed request was released"
    assert any(e[0] == "X" for e in h.events(stream)), "the error reached the request's stream before it closed"


@pytest.mark.parametrize("kind", KINDS)
def test_a_lent_slot_is_empty_and_leaves_the_prefix_tree_resident(kind):        # sync_driver.rs:317-359
    h = Harness(kind, 4, 32, 128, n_batch=16, queue_capacity=16, event_capacity=8, slow_client_timeout=0.0)
    # eight prompt tokens: a finished sequence is then long enough to stay dormant (min_prefix_len is 8)
    h.run_requests([([1, 2, 3, 4, 5, 6, 7, 8], [(3, 4)]), ([9, 10, 11, 12, 13, 14, 15, 16], [(4, 4)])])
    resident = h.kv_stats()["resident_slots"]
    assert resident > 0, "finished sequences stay dormant"
    # room beside the dormant prefixes: no eviction, an empty slot
    slot = h.lend_slot(8)
    assert slot is not None and h.seq_pos(slot) == (-1, -1)
    stats = h.kv_stats()
    assert (stats["resident_slots"], stats["evictions"]) == (resident, 0)
    # the whole pool: every dormant prefix has to make room
    slot = h.lend_slot(128)
    assert slot is not None and h.seq_pos(slot) == (-1, -1)
    stats = h.kv_stats()
    assert stats["resident_slots"] == 0 and stats["evictions"] == resident
    # more cells than the pool has: nothing left to evict
    assert h.lend_slot(129) is None


@pytest.mark.parametrize("kind", KINDS)
def test_a_slot_is_not_lent_while_a_sequence_is_live(kind):                     # sync_driver.rs:362-372
    h = sched(kind, CONTINUOUS, 16)
    stream = h.submit([1, 2, 3], [(5, 8)])            # kept: a dropped stream cancels its request
    h.pump()
    assert h.live() > 0
    with pytest.raises(h.error_type):
        h.lend_slot(1)
    assert not h.closed(stream)
