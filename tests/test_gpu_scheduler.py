"""The step scheduler driving the real engine on the GPU.

The tokens a request gets through the scheduler (continuous batching, chunked
prefill, prefix-cache copies, n > 1 groups) must be the tokens the CPU oracle
model generates for that request on its own; the scheduler's counters and
copy decisions must be those of the policy oracle run on the same request
sequence. Token ids are compared while the oracle's top-1/top-2 logit margin
exceeds 4e-2 (twice the logit tolerance)."""
import numpy as np
import pytest

import oracle
from oracle import scheduler as O
from retrograd_amd import engine as E
from retrograd_amd import scheduler as S
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPE = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                     n_ff=1024, n_vocab=1024, name="llama-q4k-sched")
N_SLOTS, N_CTX_SEQ = 4, 256


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    p = tmp_path_factory.mktemp("sched_model") / "m.gguf"
    synth.write_model(p, SHAPE, seed=321, device="cpu", std=0.05)
    return p


def oracle_greedy(model, prompt, n_new):
    """Greedy continuation by the CPU oracle, with the top-1/top-2 margin of every step."""
    ctx = oracle.Context(model, 1)
    logits = ctx.step_rows([(0, 0, list(prompt), True)])[0]
    out, margins = [], []
    pos = len(prompt)
    for _ in range(n_new):
        srt = np.sort(logits)[::-1]
        out.append(int(logits.argmax()))
        margins.append(float(srt[0] - srt[1]))
        logits = ctx.step_rows([(0, pos, [out[-1]], True)])[0]
        pos += 1
    return out, margins


def drain(stream):
    toks, end = [], None
    for e in stream.drain():
        if e.type == "Token":
            toks.append(e.token)
        elif e.type == "End":
            end = e
        else:
            raise AssertionError(e.error)
    return toks, end


def test_scheduled_requests_match_the_oracle_and_the_policy(model_path):
    print("scheduler over the engine: %s" % SHAPE.name, flush=True)
    eng = E.Engine(model_path, E.EngineConfig(n_ctx=N_SLOTS * N_CTX_SEQ, n_seq_max=N_SLOTS, n_batch=64, n_ubatch=64))
    opts = dict(mode=S.CONTINUOUS, n_batch=64, queue_capacity=32, event_capacity=256, slow_client_timeout=1.0,
                prefix_cache=True, min_prefix_len=4, swap_min_tokens=1 << 62)
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(**opts))
    sched.initialize()
    mem = eng.memory()
    assert mem.n_slots == N_SLOTS

    rng = np.random.default_rng(7)
    base = [int(t) for t in rng.integers(0, SHAPE.n_vocab, 90)]
    prompts = [
        base[:70],                                                   # cold, chunked prefill (n_batch 64)
        [int(t) for t in rng.integers(0, SHAPE.n_vocab, 9)],          # short, shares steps with the first
        base[:70] + [int(t) for t in rng.integers(0, SHAPE.n_vocab, 5)],   # extends the first: prefix hit
        base[:40],                                                   # ends inside the cached path: partial copy
        [int(t) for t in rng.integers(0, SHAPE.n_vocab, 33)],
        base[:70],                                                   # the whole prompt is cached: hit clamped to len - 1
    ]
    n_new = [6, 12, 5, 4, 7, 3]
    greedy = lambda n: E.SamplingParamsV2.greedy(max_new_tokens=n)

    # the same sequence of submissions through the policy oracle over its fake backend (same geometry)
    fake = O.FakeBackend(N_SLOTS, eng.context_size(), mem.cells_total, SHAPE.n_vocab, -1, [""] * SHAPE.n_vocab)
    policy = O.Scheduler(fake, O.Options(**{k: v for k, v in opts.items()}))
    policy.initialize()

    results = []
    waves = [[0, 1], [2], [3, 4], [5]]        # each wave runs to completion, so later waves see its prefixes
    for wave in waves:
        streams = [sched.submit(S.Request.single(prompts[i], greedy(n_new[i]))) for i in wave]
        pstreams = [policy.submit(O.Request(list(prompts[i]), [O.Sampling(max_new_tokens=n_new[i], top_k=1)])) for i in wave]
        sched.run_until_idle()
        policy.run_until_idle()
        for i, s, ps in zip(wave, streams, pstreams):
            toks, end = drain(s)
            pend = [e for e in ps.drain() if e["type"] == "End"][0]
            results.append((i, toks, end))
            assert end.reason == "MaxTokens" and len(toks) == n_new[i]
            assert end.cached_tokens == pend["cached_tokens"], (i, end.cached_tokens, pend["cached_tokens"])
    k, pk = sched.kv_stats(), policy.kv_stats()
    assert (k.hits, k.misses, k.prompt_cells, k.prefilled_cells, k.evictions, k.nodes, k.resident_slots) == \
           (pk["hits"], pk["misses"], pk["prompt_cells"], pk["prefilled_cells"], pk["evictions"], pk["nodes"],
            pk["resident_slots"])
    assert k.hits == 3 and k.misses == 3
    # the engine's occupancy is what the policy's fake pool reports: the same spans are resident
    assert eng.memory().cells_used == fake.cells_used()

    model = oracle.Model(model_path)
    compared = 0
    for i, toks, _ in results:
        want, margins = oracle_greedy(model, prompts[i], n_new[i])
        for t, w, m in zip(toks, want, margins):
            if m <= 4e-2:
                break                      # a tie within tolerance: later tokens depend on how it broke
            assert t == w, (i, toks, want)
            compared += 1
    assert compared >= 12, compared
    sched.close()
    eng.close()


def test_a_group_of_completions_prefills_once_and_samples_per_member(model_path):
    print("scheduler over the engine: n = 3 completions of one prompt", flush=True)
    eng = E.Engine(model_path, E.EngineConfig(n_ctx=N_SLOTS * N_CTX_SEQ, n_seq_max=N_SLOTS, n_batch=64, n_ubatch=64))
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=64, event_capacity=256,
                                                            prefix_cache=False))
    sched.initialize()
    rng = np.random.default_rng(11)
    prompt = [int(t) for t in rng.integers(0, SHAPE.n_vocab, 20)]
    # top_k = 40 sampling with the member's own seed; member 0 and a lone request with the same seed must agree
    def params(seed):
        return E.SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=40, seed=seed, max_new_tokens=5)
    group = sched.submit(S.Request(prompt, [params(5), params(6), params(5)]))
    sched.run_until_idle()
    by_index = {0: [], 1: [], 2: []}
    for e in group.drain():
        if e.type == "Token":
            by_index[e.index].append(e.token)
    assert all(len(v) == 5 for v in by_index.values())
    assert by_index[0] == by_index[2], "same seed, same prompt, same tokens"
    lone = sched.submit(S.Request.single(prompt, params(5)))
    sched.run_until_idle()
    lone_toks = [e.token for e in lone.drain() if e.type == "Token"]
    assert lone_toks == by_index[0], "a member of a copied group samples what a lone request samples"
    assert eng.memory().cells_used == 0
    sched.close()
    eng.close()


def test_tiny_configuration_as_specified_8_sequences_32_free_running_greedy_tokens(tmp_path):
    """The first benchmark configuration as written: the tiny Llama file (2 layers, hidden 128, 4 / 2 heads of 32,
    FFN 344, vocabulary 512, Q8_0 matrices, weights N(0, 0.02), norms 1, f16 KV), 8 sequences with prompt lengths
    uniform in [8, 64], 32 greedy tokens each, free running through the product's scheduler in continuous mode
    (no teacher forcing: each sequence is fed what the engine sampled).

    N(0, 0.02) weights give logits of spread ~0.2 whose top two are often closer than the 4e-2 a logit tolerance of
    2e-2 would call decided; the engine's actual error on this model is ~1e-5, so ids are compared wherever the
    oracle's margin exceeds 1e-3 (a hundred times that error), and at least 90 % of the 256 tokens must be compared.
    Where the margin is smaller the engine may break the tie either way; if it breaks it differently the rest of
    that sequence is no longer comparable and is left out."""
    path = tmp_path / "tiny.gguf"
    synth.write_model(path, synth.TINY_LLAMA, seed=2024, device="cpu", std=0.02)
    rng = np.random.default_rng(2024)
    lens = [int(n) for n in rng.integers(8, 65, 8)]
    prompts = [[int(t) for t in rng.integers(0, synth.TINY_LLAMA.n_vocab, n)] for n in lens]
    print("tiny configuration, prompt lengths", lens, flush=True)
    eng = E.Engine(path, E.EngineConfig(n_ctx=8 * 128, n_seq_max=8, n_batch=256, n_ubatch=256))
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=256, queue_capacity=16,
                                                            event_capacity=256, prefix_cache=False))
    sched.initialize()
    streams = [sched.submit(S.Request.single(p, E.SamplingParamsV2.greedy(seed=i, max_new_tokens=32)))
               for i, p in enumerate(prompts)]
    sched.run_until_idle()
    model = oracle.Model(path)
    compared = left_out = 0
    for i, s in enumerate(streams):
        toks, end = drain(s)
        assert end.reason == "MaxTokens" and len(toks) == 32
        want, margins = oracle_greedy(model, prompts[i], 32)
        for j, (t, w, m) in enumerate(zip(toks, want, margins)):
            if m > 1e-3:
                assert t == w, (i, j, t, w, m)
                compared += 1
            elif t != w:
                left_out += 32 - j
                break
    print("compared %d of 256 tokens, %d left out behind a tie" % (compared, left_out), flush=True)
    assert compared >= 0.9 * 256, (compared, left_out)
    assert eng.memory().cells_used == 0
    sched.close()
    eng.close()
