"""The trainer handle's generation side (include/retro_trainer.h) on the GPU: the
twins of the step surface that rollouts call (reference retro_lora_train.h:1418-1455,
1855-1945; crates/retrograd-infer/src/backend.rs:376-461).

The per-row LoRA path itself is checked against the oracle in test_gpu_lora.py. Here
the trainer is checked against it: a row that decodes under the trained adapter
(adapter 0 on a trainer) must give, bit for bit, what an engine gives for the same
row under the same file loaded as a per-row adapter; and the bookkeeping around it
(geometry of the generation context, weight changes, snapshots, the generation
default) must behave as the reference documents."""
import numpy as np
import pytest

from engine_helpers import greedy
from retrograd_amd import engine as E
from retrograd_amd import synth
from retrograd_amd import trainer as T

pytestmark = pytest.mark.gpu

SHAPE = synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                     n_ff=1024, n_vocab=1024, name="qwen2-trainer")
BASE = E.RETRO_STEP_ADAPTER_BASE


@pytest.fixture(scope="module")
def files(tmp_path_factory):
    d = tmp_path_factory.mktemp("trainer")
    model = d / "m.gguf"
    synth.write_model(model, SHAPE, seed=78, device="cpu", std=0.05)
    a1, a2 = d / "a1.gguf", d / "a2.gguf"
    synth.write_lora_adapter(a1, SHAPE, rank=16, alpha=32.0, seed=1, std_a=0.1, std_b=0.1)
    synth.write_lora_adapter(a2, SHAPE, rank=8, alpha=8.0, seed=2, std_a=0.1, std_b=0.1, targets=("attn_q", "attn_output"))
    return model, a1, a2


def trainer(model):
    return T.Trainer(model, T.TrainConfig(n_ctx=96, n_batch=96, generation_concurrency=4))


def engine(model):
    return E.Engine(model, E.EngineConfig(n_ctx=384, n_seq_max=4, n_batch=96, n_ubatch=96))


def decode(handle, prompts, adapters, n_new=3):
    """Prefill + n_new greedy steps; returns per row the tokens and the logprobs as raw bits."""
    out = E.StepOutput()
    n = len(prompts)
    for i in range(n):
        handle.seq_rm(i)            # whatever a generator call left resident
    handle.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(adapters[i]))
                 for i in range(n)], out)
    toks = [[r.token] for r in out.rows()]
    lps = [[np.float32(r.logprob).view(np.uint32)] for r in out.rows()]
    for step in range(1, n_new):
        handle.step([E.StepRow(i, i, [toks[i][-1]], len(prompts[i]) + step - 1, sample=True, sampling=greedy(),
                               adapter=E.RowAdapter(adapters[i])) for i in range(n)], out)
        for i, r in enumerate(out.rows()):
            toks[i].append(r.token)
            lps[i].append(np.float32(r.logprob).view(np.uint32))
    for i in range(n):
        handle.seq_rm(i)
        handle.request_free(i)
    return toks, lps


def test_generation_context_geometry_and_weight_changes(files):
    model, a1, a2 = files
    print("trainer: geometry and weight changes", flush=True)
    tr = trainer(model)
    mem = tr.memory()
    assert (mem.n_slots, mem.cells_total, mem.cells_used) == (4, 4 * 96, 0)     # n_ctx x generation_concurrency
    assert tr.context_size() == 96                                              # the training context's
    assert tr.kv_unified() and tr.weights_version() == 0 and not tr.is_hybrid()
    assert tr.vocab_size() == SHAPE.n_vocab
    eng = engine(model)
    assert tr.model_fingerprint() == eng.model_fingerprint()
    prompts = [[int(t) for t in np.random.default_rng(i).integers(0, SHAPE.n_vocab, n)] for i, n in enumerate((9, 17, 5))]

    # no trained adapter yet: adapter 0 is the base model
    assert decode(tr, prompts, [0, 0, 0]) == decode(eng, prompts, [0, 0, 0])

    # a weight change drops every resident cell and the generators' bookkeeping, and moves the version on
    tr.generate_continuous([(prompts[0], (1.0, 1.0, 3, 7))], 4)
    assert tr.memory().cells_used > 0 and tr.generation_stats()["calls"] == 1
    tr.load_lora(a1)
    assert tr.weights_version() == 1
    assert tr.memory().cells_used == 0 and all(tr.seq_pos(s) == (-1, -1) for s in range(4))
    tr.generate_continuous([(prompts[0] + [3], (1.0, 1.0, 2, 7))], 4)
    st = tr.generation_stats()
    assert st["calls"] == 2 and st["hits"] == 0 and st["reused_tokens"] == 0, "nothing of the old weights' KV is reused"
    for s in range(4):
        tr.seq_rm(s)

    # adapter 0 now decodes under the trained adapter, BASE under the base model - in one batch
    a1_id = eng.adapter_load(a1, 1.0)
    assert decode(tr, prompts, [0, BASE, 0]) == decode(eng, prompts, [a1_id, BASE, a1_id])
    assert decode(tr, prompts, [0, 0, 0])[0] != decode(eng, prompts, [0, 0, 0])[0], "the adapter does something"
    tr.load_lora(a2)
    assert tr.weights_version() == 2
    a2_id = eng.adapter_load(a2, 1.0)
    assert decode(tr, prompts, [0, BASE, 0]) == decode(eng, prompts, [a2_id, BASE, a2_id])
    tr.close()
    eng.close()


def test_snapshots_freeze_the_policy_and_the_generation_default_selects_one(files):
    model, a1, a2 = files
    print("trainer: snapshots and the generation default", flush=True)
    tr, eng = trainer(model), engine(model)
    with pytest.raises(E.RuntimeFailure, match="a snapshot copies the trained LoRA adapter, and the trainer has none"):
        tr.generation_adapter_snapshot()
    tr.load_lora(a1)
    snap = tr.generation_adapter_snapshot(scale=1.0)
    assert snap == 1
    info = tr.adapter_rows_info()
    assert (info.n_adapters, info.max_rank) == (1, 16), "the trained adapter itself is no per-row adapter"
    tr.load_lora(a2)                       # the policy moves on, the snapshot does not
    ids = [eng.adapter_load(a1, 1.0), eng.adapter_load(a2, 1.0)]
    prompts = [[int(t) for t in np.random.default_rng(10 + i).integers(0, SHAPE.n_vocab, n)] for i, n in enumerate((11, 6, 20))]
    assert decode(tr, prompts, [snap, 0, BASE]) == decode(eng, prompts, [ids[0], ids[1], BASE])

    # the generation default: what adapter 0 and the batched generators decode under
    assert tr.generation_adapter() == 0
    wave = [(prompts[0], (1.0, 1.0, 4, 5)), (prompts[1], (0.8, 0.9, 4, 6))]
    under_policy = tr.generate_continuous(wave, 4)
    assert tr.generation_stats()["calls"] == 1
    tr.set_generation_adapter(snap)
    assert tr.generation_adapter() == snap
    # changing it forgets the generators' bookkeeping (the same prompts are prefilled again), the KV stays
    before = tr.generation_stats()
    under_snapshot = tr.generate_continuous(wave, 4)
    after = tr.generation_stats()
    assert after["hits"] == before["hits"] and after["reused_tokens"] == before["reused_tokens"]
    assert decode(tr, prompts, [0, 0, 0]) == decode(eng, prompts, [ids[0]] * 3)
    # a second trainer whose policy is a1 generates what this one generates under the a1 snapshot
    other = trainer(model)
    other.load_lora(a1)
    want = other.generate_continuous(wave, 4)
    for (toks, lps, _), (wtoks, wlps, _) in zip(under_snapshot, want):
        assert toks == wtoks and np.array_equal(lps.view(np.uint32), wlps.view(np.uint32))
    assert [t for t, _, _ in under_policy] != [t for t, _, _ in under_snapshot]
    tr.set_generation_adapter(BASE)
    assert decode(tr, prompts, [0, 0, 0]) == decode(eng, prompts, [BASE] * 3)
    with pytest.raises(E.RuntimeFailure, match="adapter 9 is not a loaded per-row adapter"):
        tr.set_generation_adapter(9)
    with pytest.raises(E.RuntimeFailure, match="adapter -2 is not a loaded per-row adapter"):
        tr.set_generation_adapter(-2)

    # a refresh replaces the snapshot: never two at once, ids are not reused
    tr.set_generation_adapter(snap)
    newer = tr.generation_adapter_snapshot(replace=snap, scale=0.5)
    assert newer == 2 and tr.generation_adapter() == 0, "unloading the default falls back to the trained adapter"
    assert tr.adapter_rows_info().n_adapters == 1
    with pytest.raises(E.InvalidArgument, match="step row adapter 1 is not a loaded per-row adapter"):
        decode(tr, prompts[:1], [snap])
    with pytest.raises(E.RuntimeFailure, match="no per-row adapter is loaded under id 1"):
        tr.generation_adapter_unload(snap)
    tr.generation_adapter_unload(newer)
    assert tr.adapter_rows_info().n_adapters == 0
    for t in (tr, other, eng):
        t.close()


def test_rollouts_through_the_scheduler_over_a_trainer(files):
    """The scheduler over a trainer's generation context (reference backend.rs:376-461): requests decode
    under the trained adapter, and a weight change makes the scheduler let go of every cached prefix."""
    from retrograd_amd import scheduler as S
    model, a1, a2 = files
    print("trainer: scheduler over the generation context", flush=True)
    tr = trainer(model)
    tr.load_lora(a1)
    sched = S.Scheduler.over_trainer(tr, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=96, event_capacity=256,
                                                            min_prefix_len=4))
    sched.initialize()
    rng = np.random.default_rng(21)
    prompts = [[int(t) for t in rng.integers(0, SHAPE.n_vocab, n)] for n in (24, 12)]

    def run(prompt, n_new):
        stream = sched.submit(S.Request.single(prompt, E.SamplingParamsV2.greedy(max_new_tokens=n_new)))
        sched.run_until_idle()
        events = list(stream.drain())
        assert not [e for e in events if e.type == "Error"]
        return [e.token for e in events if e.type == "Token"], [e for e in events if e.type == "End"][0]

    first, end = run(prompts[0], 4)
    assert end.cached_tokens == 0
    # the same tokens as the plain step under the trained adapter gives
    eng = engine(model)
    a1_id = eng.adapter_load(a1, 1.0)
    assert first == decode(eng, [prompts[0]], [a1_id], n_new=4)[0][0]
    # a second request that extends the first reuses its cells
    again, end = run(prompts[0] + first[:2], 2)
    assert end.cached_tokens >= len(prompts[0]) and sched.kv_stats().hits == 1
    # new weights: the version moves on and nothing cached under the old ones is reused
    tr.load_lora(a2)
    assert tr.weights_version() == 2
    third, end = run(prompts[0] + first[:2], 2)
    assert end.cached_tokens == 0
    a2_id = eng.adapter_load(a2, 1.0)
    assert third == decode(eng, [prompts[0] + first[:2]], [a2_id], n_new=2)[0][0]
    sched.close()
    tr.close()
    eng.close()


def test_a_trainer_step_under_the_trained_adapter_follows_the_oracle(files):
    """The trainer handle exposes no logits, so the comparison goes through what a step returns: for every
    sampling row the ids of the eight largest logits and their log-probabilities, and the sampled token's,
    against the CPU oracle with the same adapter file loaded (prefill, then three decode steps)."""
    import oracle
    model, a1, _ = files
    print("trainer: step outputs against the oracle", flush=True)
    tr = trainer(model)
    tr.load_lora(a1)
    m = oracle.Model(model)
    aid = m.load_adapter(a1, 1.0)
    ctx = oracle.Context(m, 4)
    rng = np.random.default_rng(33)
    lens = [19, 7, 30, 12]
    prompts = [rng.integers(0, SHAPE.n_vocab, n) for n in lens]
    out = E.StepOutput(4, 8)
    feed, pos = prompts, [0] * 4
    compared = 0
    for step in range(4):
        # the whole distribution at temperature 1: the reported log-probabilities are those of the plain softmax
        tr.step([E.StepRow(i, i, feed[i], pos[i], sample=True, n_top_logprobs=8, want_logprob=True,
                           sampling=E.SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=0, seed=50 + i))
                 for i in range(4)], out)
        want = ctx.step_rows([(i, pos[i], feed[i], True) for i in range(4)], adapters=[aid] * 4).astype(np.float64)
        nxt = []
        for i in range(4):
            lp = want[i] - (np.log(np.exp(want[i] - want[i].max()).sum()) + want[i].max())
            order = np.argsort(-want[i], kind="stable")
            ids, lps = out.top(i)
            assert len(ids) == 8
            # every reported id is among the oracle's eight largest up to the tolerance, in descending order,
            # and the first one is the oracle's wherever its margin exceeds the tolerance
            assert (want[i][ids] >= want[i][order[7]] - 2 * 2e-2).all() and len(set(int(t) for t in ids)) == 8
            assert (np.diff(lps) <= 0).all()
            if want[i][order[0]] - want[i][order[1]] > 2 * 2e-2:
                assert int(ids[0]) == int(order[0])
                compared += 1
            assert np.abs(lps.astype(np.float64) - lp[ids]).max() <= 2e-2
            r = out.row(i)
            assert abs(float(r.sampled_logprob) - lp[r.token]) <= 2e-2
            nxt.append([int(r.token)])           # both sides continue with the token the trainer drew
        pos = [pos[i] + len(feed[i]) for i in range(4)]
        feed = nxt
    assert compared >= 10
    # and the adapter matters: the base model's top id differs somewhere or its log-probabilities move visibly
    base = oracle.Context(m, 4).step_rows([(i, 0, prompts[i], True) for i in range(4)])
    with_ad = oracle.Context(m, 4).step_rows([(i, 0, prompts[i], True) for i in range(4)], adapters=[aid] * 4)
    assert np.abs(base - with_ad).max() > 5e-2
    tr.close()
