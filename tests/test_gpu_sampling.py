"""The step's sampling outputs against the sampling oracle, through the C ABI.

Every case steps v2 (or v1) rows through retro_engine_step_v2, reads the f32
logits rows the step sampled from (the engine's debug hook), and feeds the same
rows, seeds and histories to oracle.sample_v2 / sample_v1 (the restatement of
reference retro_gen_core.cpp:103-225, 718-875, 2942-2985). Required:

* token ids identical over several consecutive draws of one request, which
  also checks that the request's mt19937 stream advances as the reference's
  does (one uniform draw per sampled row, seeded once);
* post-transformation top ids identical, top logprobs and sampled_logprob
  equal as floats (they come from the same double expressions);
* the temperature-1 policy logprob equal to float rounding: the device adds the
  exp terms of a row in slices, the oracle one after the other, so the double
  sum may differ in its last bits (1 ulp of the f32 result is allowed).

Rows with 0 < top_k <= 64 and no bias / penalty take the device's candidate
path (k_sample_prepare + finish_from_candidates); all others copy their logits
row to the host (sample_full_row_v2). Both are covered, also inside one step.
"""
import numpy as np
import pytest

import oracle
from retrograd_amd import engine as E
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPE = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                     n_ff=1024, n_vocab=1024, name="llama-q4k-sampling")
TIED = (17, 401, 402, 900)      # vocabulary rows given identical output weights: their logits tie bit for bit


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    from gguf_reader import Reader
    p = tmp_path_factory.mktemp("sampling") / "m.gguf"
    # std 0.2: logits spread over several units, so that top-k, min_p and top_p all cut somewhere inside the row
    synth.write_model(p, SHAPE, seed=31, device="cpu", std=0.2)
    r = Reader(p)
    ne, t, off = r.tensors["output.weight"]
    row_bytes = oracle.row_bytes(t, ne[0])
    data = bytearray(open(p, "rb").read())
    base = r.data0 + off
    src = bytes(data[base + TIED[0] * row_bytes: base + (TIED[0] + 1) * row_bytes])
    for v in TIED[1:]:
        data[base + v * row_bytes: base + (v + 1) * row_bytes] = src
    open(p, "wb").write(bytes(data))
    return p


def _engine(path, n_seq=16):
    return E.Engine(path, E.EngineConfig(n_ctx=n_seq * 128, n_seq_max=n_seq, n_batch=512, n_ubatch=512))


def _ulp_close(a, b, ulps=1):
    a, b = np.float32(a), np.float32(b)
    if a == b or (np.isinf(a) and np.isinf(b) and a == b):
        return True
    return abs(float(a) - float(b)) <= ulps * float(np.spacing(np.float32(max(abs(a), abs(b)))))


class Tracked:
    """One request on both sides: the engine's row and the oracle's generator and history."""

    def __init__(self, request, slot, prompt, params: E.SamplingParamsV2, n_top=0, want_logprob=False):
        self.request, self.slot, self.prompt = request, slot, [int(t) for t in prompt]
        self.params, self.n_top, self.want_logprob = params, n_top, want_logprob
        self.rng = oracle.Rng(params.seed)
        self.history = []
        self.pos = 0
        self.last = None

    def row(self):
        tokens = self.prompt if self.pos == 0 else [self.last]
        return E.StepRow(self.request, self.slot, tokens, self.pos, sample=True, sampling=self.params,
                         n_top_logprobs=self.n_top, want_logprob=self.want_logprob)

    def oracle_draw(self, logits):
        p = self.params
        return oracle.sample_v2(logits, self.rng, temperature=p.temperature, top_p=p.top_p, top_k=p.top_k, min_p=p.min_p,
                                repeat_penalty=p.repeat_penalty, frequency_penalty=p.frequency_penalty,
                                presence_penalty=p.presence_penalty, penalty_window=p.penalty_window,
                                bias_ids=[b[0] for b in p.logit_bias], bias_values=[b[1] for b in p.logit_bias],
                                history=self.history, k=self.n_top)

    def accept(self, token):
        n = len(self.prompt) if self.pos == 0 else 1
        self.pos += n
        self.last = int(token)
        self.history.append(int(token))


def _run(eng, tracked, n_steps, label):
    out = E.StepOutput()
    n_vocab = SHAPE.n_vocab
    for step in range(n_steps):
        print(label, "step", step, flush=True)
        eng.step([t.row() for t in tracked], out)
        logits = eng.debug_logits()
        assert logits.shape == (len(tracked), n_vocab)
        for i, t in enumerate(tracked):
            got = out.row(i)
            tok, lp, slp, ids, lps = t.oracle_draw(logits[i])
            where = (label, step, i)
            assert got.sampled and not got.forced, where
            assert got.token == tok, (where, got.token, tok)
            assert _ulp_close(got.logprob, lp), (where, got.logprob, lp)
            if t.want_logprob:
                assert np.float32(got.sampled_logprob) == np.float32(slp), (where, got.sampled_logprob, slp)
            else:
                assert got.sampled_logprob == 0.0, where
            k = min(t.n_top, n_vocab)
            assert got.n_top == k, where
            if k:
                gids, glps = out.top(i)
                assert gids.tolist() == ids.tolist(), (where, gids, ids)
                assert np.array_equal(glps, lps), (where, glps, lps)      # -inf entries included
            t.accept(tok)


def _prompts(n, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, SHAPE.n_vocab, int(rng.integers(4, 40))) for _ in range(n)]


def test_topk40_at_temperature_1_matches_the_oracle_draw_for_draw(model_path):
    """The rollout configuration's sampling: top_k 40, temperature 1, top_p 1, a seed per member."""
    eng = _engine(model_path)
    P = E.SamplingParamsV2
    tracked = [Tracked(i, i, p, P(temperature=1.0, top_p=1.0, top_k=40, seed=1000 + i, max_new_tokens=8),
                       n_top=5 if i % 2 else 0, want_logprob=bool(i % 3))
               for i, p in enumerate(_prompts(12, 3))]
    _run(eng, tracked, 8, "top_k 40")
    eng.close()


def test_candidate_path_variants_match_the_oracle(model_path):
    """Rows the device serves with (id, logit) candidates: min_p, temperature, top_p over the candidates,
    top logprobs beyond the candidate count (the -inf fill in ascending id order), greedy."""
    eng = _engine(model_path)
    P = E.SamplingParamsV2
    prompts = _prompts(8, 4)
    tracked = [
        Tracked(0, 0, prompts[0], P(temperature=0.8, top_k=64, min_p=0.05, seed=1), n_top=5, want_logprob=True),
        Tracked(1, 1, prompts[1], P(temperature=1.3, top_k=64, min_p=0.3, seed=2), n_top=64, want_logprob=True),
        Tracked(2, 2, prompts[2], P(temperature=1.0, top_k=20, top_p=0.9, seed=3), n_top=8, want_logprob=True),
        Tracked(3, 3, prompts[3], P(temperature=0.7, top_k=50, top_p=0.5, min_p=0.01, seed=4), n_top=3, want_logprob=True),
        Tracked(4, 4, prompts[4], P(temperature=1.0, top_k=3, seed=5), n_top=8, want_logprob=True),      # fill past 3
        Tracked(5, 5, prompts[5], P.greedy(seed=6), n_top=4, want_logprob=True),
        Tracked(6, 6, prompts[6], P(temperature=2.0, top_k=1, top_p=0.3, seed=7), n_top=2),
        Tracked(7, 7, prompts[7], P(temperature=1.0, top_k=2, top_p=1e-6, seed=8), n_top=5, want_logprob=True),
    ]
    _run(eng, tracked, 6, "candidates")
    eng.close()


def test_full_row_path_matches_the_oracle(model_path):
    """Rows that sample from a host copy of the logits: no top_k, top_k above the device limit, top_p alone,
    logit bias, penalties with and without a window (the history is what the request sampled so far)."""
    eng = _engine(model_path)
    P = E.SamplingParamsV2
    prompts = _prompts(9, 5)
    bias = [(7, 6.0), (8, -50.0), (300, 2.5), (1023, 4.0)]
    tracked = [
        Tracked(0, 0, prompts[0], P(temperature=1.0, top_p=0.9, top_k=0, seed=11), n_top=5, want_logprob=True),
        Tracked(1, 1, prompts[1], P(temperature=0.9, top_p=1.0, top_k=0, seed=12), n_top=3, want_logprob=True),
        Tracked(2, 2, prompts[2], P(temperature=1.0, top_k=100, seed=13), n_top=10, want_logprob=True),   # > 64
        Tracked(3, 3, prompts[3], P(temperature=1.0, top_k=40, seed=14, logit_bias=bias), n_top=6, want_logprob=True),
        Tracked(4, 4, prompts[4], P(temperature=1.0, top_k=10, seed=15, repeat_penalty=1.3, frequency_penalty=0.4,
                                    presence_penalty=0.2, penalty_window=3), n_top=5, want_logprob=True),
        Tracked(5, 5, prompts[5], P(temperature=0.6, top_k=5, seed=16, repeat_penalty=1.5), n_top=5, want_logprob=True),
        Tracked(6, 6, prompts[6], P(temperature=1.0, top_k=0, min_p=0.2, seed=17, presence_penalty=1.0,
                                    logit_bias=[(5, 3.0)]), n_top=4),
        Tracked(7, 7, prompts[7], P(temperature=1.0, top_k=SHAPE.n_vocab, seed=18), n_top=2, want_logprob=True),  # k = V: no cut
        Tracked(8, 8, prompts[8], P(temperature=1.0, top_k=1, seed=19, frequency_penalty=2.0), n_top=3, want_logprob=True),
    ]
    _run(eng, tracked, 7, "full row")
    eng.close()


def test_both_paths_in_one_step_and_a_request_that_changes_its_parameters(model_path):
    """Candidate rows and full rows share a step; a request may change parameters between steps (the generator
    and the history stay the request's)."""
    eng = _engine(model_path)
    P = E.SamplingParamsV2
    prompts = _prompts(4, 6)
    tracked = [
        Tracked(0, 0, prompts[0], P(temperature=1.0, top_k=40, seed=21), n_top=5, want_logprob=True),
        Tracked(1, 1, prompts[1], P(temperature=1.0, top_k=0, top_p=0.95, seed=22), n_top=5, want_logprob=True),
        Tracked(2, 2, prompts[2], P(temperature=1.0, top_k=40, seed=23, repeat_penalty=1.2)),
        Tracked(3, 3, prompts[3], P.greedy(seed=24)),
    ]
    _run(eng, tracked, 3, "mixed a")
    tracked[0].params = P(temperature=1.0, top_k=0, top_p=0.8, seed=999, presence_penalty=0.5)   # seed ignored: already seeded
    tracked[1].params = P(temperature=0.5, top_k=8, seed=999)
    _run(eng, tracked, 3, "mixed b")
    eng.close()


def test_ties_inside_and_at_the_edge_of_the_top_k(model_path):
    """Four vocabulary rows share their output weights, so their logits are equal bit for bit. A bias lifts the
    tied group to the top (full-row path); without a bias the candidate path meets the tie wherever the model
    puts it. top-logprob order among equal weights is ascending id on both sides (retro_gen_core.cpp:857-862)."""
    eng = _engine(model_path)
    out = E.StepOutput()
    P = E.SamplingParamsV2
    prompt = _prompts(1, 7)[0]
    eng.step([E.StepRow(0, 0, prompt, 0, sample=True, sampling=P.greedy())], out)
    logits = eng.debug_logits()[0]
    assert len({logits[v].tobytes() for v in TIED}) == 1, "the tied rows must produce identical logits"
    eng.seq_rm(0)
    eng.request_free(0)
    # how far below the maximum the tied value sits decides the bias that makes it the top value
    lift = float(logits.max() - logits[TIED[0]]) + 1.0
    bias = [(v, lift) for v in TIED]
    tracked = [
        # the tied group is the whole top 4; top_k = 4 keeps exactly it, n_top lists it by ascending id
        Tracked(1, 1, prompt, P(temperature=1.0, top_k=4, seed=31, logit_bias=bias), n_top=6, want_logprob=True),
        # top_k = 8 with the tie inside
        Tracked(2, 2, prompt, P(temperature=1.0, top_k=8, seed=32, logit_bias=bias), n_top=8, want_logprob=True),
        # greedy over a tied maximum: argmax takes the lowest id, as partial_sort's first element does
        Tracked(3, 3, prompt, P(temperature=1.0, top_k=1, seed=33, logit_bias=bias), n_top=2, want_logprob=True),
    ]
    _run(eng, tracked, 3, "ties, bias")
    # candidate path: rank of the tied value in this row decides a top_k that cuts right behind / inside the group
    rank = int((logits > logits[TIED[0]]).sum())
    # (a row whose cut falls inside a run of equal logits, or whose nucleus sorts equal weights, is fetched and
    # sampled by the full-row code: which of the equal entries survive is std::partial_sort's / std::sort's doing)
    if rank + 4 <= 64:
        tracked = [
            Tracked(4, 4, prompt, P(temperature=1.0, top_k=rank + 4, seed=34), n_top=rank + 4, want_logprob=True),
            Tracked(5, 5, prompt, P(temperature=1.0, top_k=rank + 2, seed=35), n_top=rank + 4, want_logprob=True),
            Tracked(6, 6, prompt, P(temperature=1.0, top_k=rank + 1, seed=36), n_top=3, want_logprob=True),
            Tracked(7, 7, prompt, P(temperature=1.0, top_k=rank + 4, top_p=0.97, seed=37), n_top=rank + 4, want_logprob=True),
            Tracked(8, 8, prompt, P(temperature=1.0, top_k=rank + 3, top_p=0.5, seed=38), n_top=4, want_logprob=True),
        ]
        _run(eng, tracked, 2, "ties, candidates")
    eng.close()


def test_v1_rows_report_the_oracles_logprobs_and_top_logprobs(model_path):
    """v1 rows (temperature + top_p): token, logprob and the raw temperature-1 top-k logprobs
    (retro_gen_core.cpp:2958-2985) against the oracle."""
    eng = _engine(model_path)
    prompts = _prompts(3, 8)
    settings = [(1.0, 1.0, 41), (0.7, 0.9, 42), (1.5, 0.5, 43)]
    rngs = [oracle.Rng(s[2]) for s in settings]
    pos = [0, 0, 0]
    last = [None] * 3
    for step in range(4):
        print("v1 step", step, flush=True)
        rows = []
        for i, p in enumerate(prompts):
            toks = [int(t) for t in p] if step == 0 else [last[i]]
            t, tp, seed = settings[i]
            rows.append((i, i, toks, pos[i], True, t, tp, seed, 4))
        res, top_ids, top_lps = eng.step_v1(rows, n_top_stride=4)
        logits = eng.debug_logits()
        for i in range(3):
            t, tp, _ = settings[i]
            tok, lp, ids, lps = oracle.sample_v1(logits[i], t, tp, rngs[i], k=4)
            assert res[i].token == tok, (step, i)
            assert _ulp_close(res[i].logprob, lp, ulps=2), (step, i, res[i].logprob, lp)
            assert top_ids[i].tolist() == ids.tolist(), (step, i)
            assert all(_ulp_close(a, b, ulps=2) for a, b in zip(top_lps[i], lps)), (step, i, top_lps[i], lps)
            pos[i] += len(rows[i][2])
            last[i] = tok
    eng.close()
