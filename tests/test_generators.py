"""The oracle of the batched generators (oracle/generate.py) against the
reference's own scenarios and hand-derived counters, over a synthetic backend
whose logits are a closed form of a row's history (no model, no GPU).

Scenarios and expected values come from the reference:
tests/engine_runtime.rs:294-306 (calls/sequences after one call), :362-404
(budgets bounded by the context, dormant prefixes evicted), :676-724 (a wave
with a shared prompt), tests/grpo_runtime.rs (multi-turn reuse counters) and the
contract text of retro_gen_core.cpp:317-331 (permuting the caller's rows only
permutes the outputs)."""
import zlib

import numpy as np
import pytest

from oracle import generate as G

V = 64


class HistoryBackend:
    """Per-slot token lists; the logits of a row are a pseudo-random function
    of everything resident in the slot up to and including the row's token."""

    def __init__(self, n_slots):
        self.kv = [[] for _ in range(n_slots)]
        self.decoded_positions = 0

    def decode(self, rows):
        out = []
        for slot, pos0, tokens, want in rows:
            assert len(self.kv[slot]) == pos0, "positions must stay consecutive"
            self.kv[slot].extend(int(t) for t in tokens)
            self.decoded_positions += len(tokens)
            if want:
                seed = zlib.crc32(np.asarray(self.kv[slot], np.int32).tobytes())
                out.append(np.random.default_rng(seed).standard_normal(V).astype(np.float32) * 3.0)
        return out

    def seq_rm(self, slot, p0, p1):
        assert (p0, p1) == (-1, -1)
        self.kv[slot] = []

    def seq_cp(self, src, dst, p0, p1):
        assert (p0, p1) == (-1, -1) and not self.kv[dst]
        self.kv[dst] = list(self.kv[src])


def make(n_seq_max=4, n_batch=8, n_ctx=256, n_ctx_seq=None, eog=()):
    be = HistoryBackend(n_seq_max)
    gen = G.Generator(be, n_seq_max=n_seq_max, n_batch=n_batch, n_ctx=n_ctx, n_ctx_seq=n_ctx_seq or n_ctx, n_vocab=V, eog=eog)
    return gen, be


def p(seed, max_new=6, temperature=1.0, top_p=1.0):
    return (temperature, top_p, max_new, seed)


def test_canonical_order_is_length_then_tokens_then_sampling():
    seqs = [([5, 6, 7], p(3)), ([5, 6], p(9)), ([5, 6, 7], p(1)), ([4, 9, 9], p(2)), ([5, 6, 7], p(1, max_new=2))]
    assert G.canonical_order(seqs) == [1, 3, 4, 2, 0]
    # equal rows keep the caller's order (stable sort)
    assert G.canonical_order([([1], p(1)), ([1], p(1))]) == [0, 1]


def test_one_call_counts_one_call_and_its_sequences():
    gen, _ = make()
    assert gen.stats.calls == 0
    gen.generate_continuous_batch([([1, 2, 3, 4], p(7))], 6)
    assert gen.stats.calls == 1 and gen.stats.sequences == 1
    assert gen.stats.prompt_tokens == 4 and gen.stats.prefilled_tokens == 4 and gen.stats.reused_tokens == 0


def test_wave_with_a_shared_prompt_prefills_it_once_and_copies():
    gen, be = make(n_batch=8)
    first, second = [10, 11, 12, 13, 14], [20, 21, 22, 23]
    wave = [(second, p(50)), (first, p(51)), (first, p(52))]
    out = gen.generate_continuous_batch(wave, 6)
    assert [len(t) for t, _ in out] == [6, 6, 6]
    # canonical order: `second` (shorter) first, in its own launch; then the prefix of `first` once,
    # the copy, and one terminal row per member
    assert gen.launches[0] == [(0, 0, 4, True)]
    assert gen.launches[1] == [(1, 0, 4, False)]
    assert gen.launches[2] == [(1, 4, 1, True), (2, 4, 1, True)]
    assert gen.stats.prefilled_tokens == 4 + 4 + 2 and gen.stats.prompt_tokens == 4 + 5 + 5
    # every decode launch carries the live rows in canonical order
    assert gen.launches[3] == [(0, 4, 1, True), (1, 5, 1, True), (2, 5, 1, True)]
    # members of the copy group differ only by their seeds
    assert out[1][0] != out[2][0]


def test_permuting_the_rows_only_permutes_the_outputs():
    wave = [([3, 4, 5], p(1)), ([9, 8, 7, 6], p(2)), ([3, 4, 5], p(3)), ([1], p(4))]
    gen, _ = make()
    base = gen.generate_continuous_batch(wave, 5)
    for perm in ([2, 0, 3, 1], [3, 2, 1, 0]):
        g2, _ = make()
        got = g2.generate_continuous_batch([wave[i] for i in perm], 5)
        for k, i in enumerate(perm):
            assert got[k][0] == base[i][0] and np.array_equal(got[k][1], base[i][1])


def test_a_later_turn_decodes_only_the_extension():
    gen, be = make()
    prompt = [1, 2, 3, 4, 5]
    (tokens, _), = gen.generate_continuous_batch([(prompt, p(5, max_new=4))], 8)
    assert gen.slots[0] == prompt + tokens[:-1], "the last emitted token is never fed back"
    before = gen.stats.as_dict()
    turn2 = prompt + tokens + [7, 8]
    gen.generate_continuous_batch([(turn2, p(6, max_new=3))], 8)
    d = {k: gen.stats.as_dict()[k] - before[k] for k in before}
    resident = len(prompt) + len(tokens) - 1
    assert d == {"calls": 1, "sequences": 1, "prompt_tokens": len(turn2), "prefilled_tokens": len(turn2) - resident,
                 "reused_tokens": resident, "hits": 1, "evictions": 0}
    # a prompt that diverges goes to a slot that holds nothing, while there is one: the warm slot survives
    before = gen.stats.as_dict()
    gen.generate_continuous_batch([([1, 2, 9, 9], p(7, max_new=2))], 8)
    d = {k: gen.stats.as_dict()[k] - before[k] for k in before}
    assert d["hits"] == 0 and d["evictions"] == 0 and d["prefilled_tokens"] == 4 and d["reused_tokens"] == 0
    assert gen.slots[0][:5] == prompt and gen.slots[1][:4] == [1, 2, 9, 9]
    # with a single slot the divergence costs the slot
    g1, _ = make(n_seq_max=1)
    g1.generate_continuous_batch([(prompt, p(5, max_new=4))], 8)
    g1.generate_continuous_batch([([1, 2, 9, 9], p(7, max_new=2))], 8)
    assert g1.stats.hits == 0 and g1.stats.evictions == 1
    # a resident block as long as the prompt is not a hit: the terminal position must be decoded by this call
    gen2, _ = make(n_seq_max=1)
    gen2.generate_continuous_batch([(prompt, p(1, max_new=1))], 4)
    assert gen2.slots[0] == prompt
    gen2.generate_continuous_batch([(prompt, p(2, max_new=1))], 4)
    assert gen2.stats.hits == 0 and gen2.stats.evictions == 1 and gen2.stats.prefilled_tokens == 10


def test_the_least_recently_extended_slot_is_sacrificed():
    gen, _ = make(n_seq_max=2)
    gen.generate_continuous_batch([([1, 1, 1], p(1, max_new=2))], 4)          # slot 0, clock 1
    gen.generate_continuous_batch([([2, 2, 2], p(1, max_new=2))], 4)          # slot 1 (empty, used_at 0 < 1), clock 2
    assert gen.slots[0][:3] == [1, 1, 1] and gen.slots[1][:3] == [2, 2, 2]
    gen.generate_continuous_batch([([3, 3, 3], p(1, max_new=2))], 4)          # sacrifices slot 0 (older)
    assert gen.slots[0][:3] == [3, 3, 3] and gen.slots[1][:3] == [2, 2, 2]
    assert gen.stats.evictions == 1


def test_large_budgets_are_bounded_by_the_context_and_dormant_prefixes_yield():
    # reference tests/engine_runtime.rs:362-404: n_ctx 256, two slots, prompts of 252 and 250 tokens
    gen, _ = make(n_seq_max=2, n_batch=64, n_ctx=256)
    unlimited, u32max = p(2, max_new=2**32 - 1), 2**32 - 1
    for length in (252, 250):
        prompt = [1] * length
        g_b, _ = make(n_seq_max=2, n_batch=64, n_ctx=256)
        bounded = g_b.generate_continuous_batch([(prompt, p(2, max_new=256 - length))], u32max and 8)
        got = gen.generate_continuous_batch([(prompt, unlimited)], 8)
        assert got[0][0] == bounded[0][0] and len(got[0][0]) == min(8, 256 - length)
    assert gen.stats.evictions > 0, "dormant near-full prefixes must yield their KV cells to the next call"


def test_generate_batch_decodes_the_prompt_once_and_members_draw_from_the_same_row():
    gen, be = make(n_batch=4)
    prompt = [1, 2, 3, 4, 5, 6]
    out = gen.generate_batch(prompt, [p(61, 5), p(62, 5), p(61, 5)], 5)
    assert gen.launches[0] == [(0, 0, 4, False)] and gen.launches[1] == [(0, 4, 2, True)]
    assert out[0][0] == out[2][0] and np.array_equal(out[0][1], out[2][1]), "same seed, same tokens"
    assert out[0][0] != out[1][0]
    assert all(not kv for kv in be.kv), "the call leaves an empty context"
    # a member of generate_batch and a lone continuous row with the same seed agree
    g2, _ = make(n_batch=4)
    lone = g2.generate_continuous_batch([(prompt, p(62, 5))], 5)
    assert lone[0][0] == out[1][0] and np.array_equal(lone[0][1], out[1][1])


def test_end_of_generation_tokens_stop_a_row_and_are_included():
    gen, _ = make()
    base = gen.generate_continuous_batch([([1, 2, 3], p(3, max_new=6))], 6)[0][0]
    stop = base[2]
    g2, _ = make(eog=(stop,))
    got = g2.generate_continuous_batch([([1, 2, 3], p(3, max_new=6))], 6)[0][0]
    assert got == base[:base.index(stop) + 1]


def test_argument_errors_carry_the_reference_messages():
    gen, _ = make(n_seq_max=2, n_batch=2)
    with pytest.raises(G.GenerationError, match="generation batch has 3 sequences but the context supports 2"):
        gen.generate_batch([1], [p(1), p(2), p(3)], 4)
    with pytest.raises(G.GenerationError, match="exceeds the configured sequence or batch capacity"):
        gen.generate_continuous_batch([([1], p(1)), ([1], p(2)), ([1], p(3))], 4)
    with pytest.raises(G.GenerationError, match="temperature must be finite and greater than zero"):
        gen.generate_batch([1], [p(1, temperature=0.0)], 4)
    with pytest.raises(G.GenerationError, match="top_p must be in"):
        gen.generate_continuous_batch([([1], p(1, top_p=0.0))], 4)
    with pytest.raises(G.GenerationError, match="token 64 at index 1 is outside the vocabulary of size 64"):
        gen.generate_batch([1, 64], [p(1)], 4)
    with pytest.raises(G.GenerationError, match="prompt of 256 tokens leaves no room to generate in context 256"):
        gen.generate_batch([1] * 256, [p(1)], 4)


def test_the_reuse_can_be_switched_off(monkeypatch):
    monkeypatch.setenv("RETRO_GENERATION_PREFIX_CACHE", "0")
    gen, be = make()
    gen.generate_continuous_batch([([1, 2, 3], p(1, max_new=2)), ([4, 5], p(2, max_new=2))], 4)
    assert all(not kv for kv in be.kv) and gen.stats.calls == 1 and gen.stats.sequences == 0
    # caller slots, not placement: row i lives in slot i
    assert gen.launches[0] == [(1, 0, 2, True)] and gen.launches[1] == [(0, 0, 3, True)]
