"""The batched generators of the C ABI (retro_engine_generate_batch,
retro_engine_generate_continuous_batch, retro_engine_generation_stats) on the GPU.

Against the oracle (oracle/generate.py over the CPU forward pass): tokens,
log-probabilities, the reuse counters and what every slot holds after each call.
And the reference's own relational tests, replayed on this build: a caller-side
loop over the step in canonical order reproduces the continuous generator bit
for bit (tests/engine_runtime.rs:676-724), a lockstep wave through the scheduler
does (tests/infer_runtime.rs:90-154), and a request with n = 3 completions
matches generate_batch in tokens and log-probabilities
(tests/infer_runtime.rs:156-197)."""
import numpy as np
import pytest

import oracle
from oracle import generate as G
from retrograd_amd import engine as E
from retrograd_amd import scheduler as S
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPE = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                     n_ff=1024, n_vocab=1024, name="llama-q4k-gen")
N_SLOTS, N_CTX, N_BATCH = 4, 4 * 96, 16


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    p = tmp_path_factory.mktemp("gen_model") / "m.gguf"
    synth.write_model(p, SHAPE, seed=77, device="cpu", std=0.05)
    return p


def engine(model_path, n_slots=N_SLOTS, n_ctx=N_CTX, n_batch=N_BATCH):
    return E.Engine(model_path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_slots, n_batch=n_batch, n_ubatch=n_batch))


def oracle_generator(model_path, n_slots=N_SLOTS, n_ctx=N_CTX, n_batch=N_BATCH):
    model = oracle.Model(model_path)
    ctx = oracle.Context(model, n_slots)
    return G.Generator(G.ContextBackend(ctx), n_seq_max=n_slots, n_batch=n_batch, n_ctx=n_ctx, n_ctx_seq=n_ctx,
                       n_vocab=SHAPE.n_vocab, eog=())


def p(seed, max_new=6, temperature=1.0, top_p=1.0):
    return (temperature, top_p, max_new, seed)


def prompts(seed, lengths):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, SHAPE.n_vocab, n)] for n in lengths]


def assert_same_generation(got, want, lp_tol=2e-3):
    assert len(got) == len(want)
    for (toks, lps, forced), (wtoks, wlps) in zip(got, want):
        assert toks == wtoks
        assert not any(forced)
        assert np.abs(lps - wlps).max() <= lp_tol


def test_continuous_generation_matches_the_oracle_call_after_call(model_path):
    print("continuous generator vs oracle", flush=True)
    eng, orc = engine(model_path), oracle_generator(model_path)
    first, second, third = prompts(1, [9, 7, 12])
    # a wave with a shared prompt, submitted out of canonical order
    wave = [(second, p(50)), (first, p(51)), (first, p(52, max_new=4))]
    got = eng.generate_continuous(wave, 8)
    want = orc.generate_continuous_batch(wave, 8)
    assert_same_generation(got, want)
    assert eng.generation_stats() == orc.stats.as_dict()
    assert eng.generation_stats()["prefilled_tokens"] == 7 + 8 + 2
    # what the slots hold: the prompt and every sampled token but the last
    for slot in range(N_SLOTS):
        lo_hi = eng.seq_pos(slot)
        assert lo_hi == ((0, len(orc.slots[slot]) - 1) if orc.slots[slot] else (-1, -1)), slot
    # second turn: two rows extend what their slots hold, one is new
    turn = [(first + got[1][0] + [3, 4], p(60, max_new=3)), (third, p(61, max_new=5)), (second + got[0][0] + [5], p(62, max_new=2))]
    got2 = eng.generate_continuous(turn, 8)
    want2 = orc.generate_continuous_batch(turn, 8)
    assert_same_generation(got2, want2)
    st = eng.generation_stats()
    assert st == orc.stats.as_dict()
    assert st["hits"] == 2 and st["calls"] == 2 and st["evictions"] == 0
    assert st["reused_tokens"] == (9 + 6 - 1) + (7 + 6 - 1)
    for slot in range(N_SLOTS):
        assert eng.seq_pos(slot) == ((0, len(orc.slots[slot]) - 1) if orc.slots[slot] else (-1, -1)), slot
    # a raw sequence operation through the ABI forgets what the slots hold: the next call starts cold
    eng.seq_rm(3)
    before = eng.generation_stats()
    eng.generate_continuous([(first + got[1][0] + [3, 4] + got2[0][0] + [9], p(70, max_new=2))], 8)
    after = eng.generation_stats()
    assert after["hits"] == before["hits"] and after["reused_tokens"] == before["reused_tokens"]
    eng.close()


def test_generate_batch_matches_the_oracle(model_path):
    print("generate_batch vs oracle", flush=True)
    eng, orc = engine(model_path), oracle_generator(model_path)
    (prompt,) = prompts(2, [21])          # longer than n_batch: the prefix takes two launches
    sampling = [p(61, 5), p(62, 5, temperature=0.7, top_p=0.9), p(61, 5)]
    got = eng.generate_batch(prompt, sampling, 6)
    want = orc.generate_batch(prompt, sampling, 6)
    assert_same_generation(got, want)
    assert got[0][0] == got[2][0] and np.array_equal(got[0][1], got[2][1]), "same seed, same tokens and logprobs"
    assert eng.memory().cells_used == 0, "the call leaves an empty context"
    assert eng.generation_stats()["calls"] == 0, "only the continuous path counts calls"
    eng.close()


def canonical_step_loop(eng, sequences, n_batch):
    """The caller-side loop of the reference's tests/engine_runtime.rs:533-675:
    prompts prefilled through the step in canonical order (chunks of n_batch,
    equal prompts decoded once and copied), then one step per wave over the
    live rows, in canonical order."""
    n_ctx_seq = eng.context_size()
    order = G.canonical_order(sequences)
    slot_of = {seq: slot for slot, seq in enumerate(order)}
    for slot in range(len(order)):
        eng.seq_rm(slot)
    tokens = {s: [] for s in order}
    lps = {s: [] for s in order}
    nxt = {}

    def row(seq, toks, pos0, sample):
        temperature, top_p, _, seed = sequences[seq][1]
        return (seq + 1, slot_of[seq], toks, pos0, sample, temperature, top_p, seed, 0)

    g = 0
    while g < len(order):
        leader = order[g]
        prompt = sequences[leader][0]
        e = g + 1
        while e < len(order) and sequences[order[e]][0] == prompt:
            e += 1
        members = order[g:e]
        if len(members) > 1:
            for at in range(0, len(prompt) - 1, n_batch):
                eng.step_v1([row(leader, prompt[at:min(at + n_batch, len(prompt) - 1)], at, False)])
            for m in members[1:]:
                eng.seq_cp(slot_of[leader], slot_of[m])
            outs, _, _ = eng.step_v1([row(m, [prompt[-1]], len(prompt) - 1, True) for m in members])
            for m, o in zip(members, outs):
                nxt[m] = o
        else:
            for at in range(0, len(prompt), n_batch):
                chunk = prompt[at:at + n_batch]
                last = at + len(chunk) == len(prompt)
                outs, _, _ = eng.step_v1([row(leader, chunk, at, last)])
                if last:
                    nxt[leader] = outs[0]
        g = e
    limits = {s: min(sequences[s][1][2], n_ctx_seq - len(sequences[s][0])) for s in order}
    live = set(order)
    while live:
        active = []
        for s in order:
            if s not in live:
                continue
            tokens[s].append(nxt[s].token)
            lps[s].append(np.float32(nxt[s].logprob))
            if eng.is_eog_token(nxt[s].token) or len(tokens[s]) == limits[s]:
                live.discard(s)
            else:
                active.append(s)
        if not active:
            break
        outs, _, _ = eng.step_v1([row(s, [tokens[s][-1]], len(sequences[s][0]) + len(tokens[s]) - 1, True) for s in active])
        for s, o in zip(active, outs):
            nxt[s] = o
    for s in order:
        eng.request_free(s + 1)
    return [(tokens[s], np.array(lps[s], np.float32)) for s in range(len(sequences))]


def test_a_step_loop_in_canonical_order_reproduces_the_continuous_generator_bit_for_bit(model_path):
    print("step loop vs generator", flush=True)
    eng = engine(model_path)
    first, second = prompts(3, [11, 8])
    wave = [(second, p(50)), (first, p(51)), (first, p(52))]
    reference = eng.generate_continuous(wave, 6)
    stepped = canonical_step_loop(eng, wave, N_BATCH)
    for (toks, lps, _), (stoks, slps) in zip(reference, stepped):
        assert toks == stoks
        assert np.array_equal(lps.view(np.uint32), slps.view(np.uint32)), "logprobs bit for bit"
    # the per-token logprobs also match the single-prompt batched generator
    for index, (prompt, sampling) in enumerate(wave):
        alone = eng.generate_batch(prompt, [sampling], 6)[0]
        assert alone[0] == stepped[index][0]
        assert np.array_equal(alone[1].view(np.uint32), stepped[index][1].view(np.uint32))
    eng.close()


def drain(stream, index=0):
    toks, lps, end = [], [], None
    for e in stream.drain():
        if e.type == "Token" and e.index == index:
            toks.append(e.token)
            lps.append(np.float32(e.logprob))
        elif e.type == "End" and e.index == index:
            end = e
        elif e.type == "Error":
            raise AssertionError(e.error)
    return toks, np.array(lps, np.float32), end


def test_the_scheduler_matches_the_generators_bit_for_bit(model_path):
    print("scheduler vs generators", flush=True)
    ref = engine(model_path)
    first, second = prompts(4, [10, 7])
    wave = [(second, p(50)), (first, p(51)), (first, p(52))]
    reference = ref.generate_continuous(wave, 6)
    prompt = first
    sampling = [p(61, 5), p(62, 5), p(63, 5)]
    batch_reference = ref.generate_batch(prompt, sampling, 5)
    ref.close()

    def v2(params):
        temperature, top_p, max_new, seed = params
        return E.SamplingParamsV2(temperature=temperature, top_p=top_p, seed=seed, max_new_tokens=max_new)

    # a lockstep wave of single requests = the continuous generator
    eng = engine(model_path)
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.LOCKSTEP, n_batch=N_BATCH, event_capacity=256))
    sched.initialize()
    streams = [sched.submit(S.Request.single(list(pr), v2(sp))) for pr, sp in wave]
    sched.run_until_idle()
    for index, stream in enumerate(streams):
        toks, _, end = drain(stream)
        assert toks == reference[index][0], "request %d: tokens bit for bit" % index
        assert end.reason == "MaxTokens"
    sched.close()
    eng.close()

    # one request with three completions = generate_batch, log-probabilities included
    eng = engine(model_path)
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=N_BATCH, event_capacity=256))
    sched.initialize()
    stream = sched.submit(S.Request(list(prompt), [v2(sp) for sp in sampling]))
    sched.run_until_idle()
    events = list(stream.drain())
    for index, (wtoks, wlps, _) in enumerate(batch_reference):
        toks = [e.token for e in events if e.type == "Token" and e.index == index]
        lps = np.array([e.logprob for e in events if e.type == "Token" and e.index == index], np.float32)
        assert toks == wtoks, "member %d: tokens" % index
        assert np.array_equal(lps.view(np.uint32), wlps.view(np.uint32)), "member %d: logprobs bit for bit" % index
    sched.close()
    eng.close()


def test_budgets_are_bounded_by_the_context_and_dormant_prefixes_yield(model_path):
    # reference tests/engine_runtime.rs:362-404, on a 256-cell pool with two slots
    print("context-bounded budgets", flush=True)
    eng = engine(model_path, n_slots=2, n_ctx=256, n_batch=64)
    for length in (252, 250):
        prompt = [1] * length
        bounded = eng.generate_continuous([(prompt, p(2, max_new=256 - length))], 8)
        unlimited = eng.generate_continuous([(prompt, p(2, max_new=2**32 - 1))], 8)
        assert unlimited[0][0] == bounded[0][0] and len(unlimited[0][0]) == min(8, 256 - length)
        assert np.array_equal(unlimited[0][1], bounded[0][1])
    assert eng.generation_stats()["evictions"] > 0, "dormant near-full prefixes must yield their KV cells to the next call"
    eng.close()


def test_argument_errors(model_path):
    eng = engine(model_path, n_slots=2, n_ctx=64, n_batch=2)
    with pytest.raises(E.RuntimeFailure, match="generation batch has 3 sequences but the context supports 2"):
        eng.generate_batch([1], [p(1), p(2), p(3)], 4)
    with pytest.raises(E.RuntimeFailure, match="exceeds the configured sequence or batch capacity"):
        eng.generate_continuous([([1], p(1)), ([1], p(2)), ([1], p(3))], 4)
    with pytest.raises(E.RuntimeFailure, match="temperature must be finite and greater than zero"):
        eng.generate_batch([1], [p(1, temperature=0.0)], 4)
    with pytest.raises(E.RuntimeFailure, match="token 1024 at index 1 is outside the vocabulary of size 1024"):
        eng.generate_batch([1, 1024], [p(1)], 4)
    with pytest.raises(E.RuntimeFailure, match="prompt of 64 tokens leaves no room to generate in context 64"):
        eng.generate_batch([1] * 64, [p(1)], 4)
    with pytest.raises(E.RuntimeFailure, match="top_p must be in"):
        eng.generate_continuous([([1], p(1, top_p=1.5))], 4)
    assert eng.generate_batch([1], [p(1, max_new=2), p(2, max_new=2)], 4)[0][0]
    eng.close()


def test_prefix_cache_reuse_matches_cold_generation(model_path):
    """reference tests/infer_runtime.rs:243-329: requests served from the scheduler's prefix tree (a partial
    copy of a shared prefix; a fully cached prompt served by replaying its last token) generate what the
    continuous generator generates cold. The reference asserts it bit for bit on its CPU path; here the
    warm path prefills a suffix where the cold path prefills the whole prompt, in launches of another
    shape, so the logits agree to accumulation order and the sampled tokens are compared."""
    print("prefix cache warm vs cold", flush=True)
    config = E.EngineConfig(n_ctx=256, n_seq_max=4, n_batch=64, n_ubatch=64)
    ref = E.Engine(model_path, config)
    rng = np.random.default_rng(31)
    shared = [int(t) for t in rng.integers(0, SHAPE.n_vocab, 96)]
    suffix_a, suffix_b = ([int(t) for t in rng.integers(0, SHAPE.n_vocab, n)] for n in (5, 6))
    prompt_a = shared + suffix_a
    ref_a = ref.generate_continuous([(prompt_a, p(81, 5))], 5)
    wave2 = [(shared + suffix_b, p(82, 5)), (shared, p(83, 5))]
    ref_b = ref.generate_continuous(wave2, 5)
    ref.close()

    def v2(params):
        temperature, top_p, max_new, seed = params
        return E.SamplingParamsV2(temperature=temperature, top_p=top_p, seed=seed, max_new_tokens=max_new)

    eng = E.Engine(model_path, config)
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.LOCKSTEP, n_batch=64, queue_capacity=16, event_capacity=256))
    sched.initialize()
    stream = sched.submit(S.Request.single(prompt_a, v2(p(81, 5))))
    sched.run_until_idle()
    toks, _, _ = drain(stream)
    assert toks == ref_a[0][0]
    assert sched.kv_stats().nodes == 1
    streams = [sched.submit(S.Request.single(prompt, v2(sampling))) for prompt, sampling in wave2]
    sched.run_until_idle()
    for index, stream in enumerate(streams):
        toks, _, end = drain(stream)
        assert toks == ref_b[index][0], "wave 2 request %d (request 1 is a full-prompt hit)" % index
        assert end.cached_tokens == (96 if index == 0 else 95)
    assert sched.kv_stats().hits == 2
    sched.close()
    eng.close()
