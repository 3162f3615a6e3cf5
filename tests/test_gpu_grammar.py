"""Grammar-constrained sampling rows through the C ABI (reference retro_gen_core.cpp:767-795, 2518-2537, 2688-2710,
2738; grammar handles retro_lora_train.h:1395-1408).

The reference's own scenarios with their expected values: an invalid grammar is refused before anything decodes,
`root ::= <[id]>` forces a token with sampled_logprob 0, and a later row of the request without a grammar samples
freely again (tests/engine_runtime.rs:1078-1140); two rows of one call keep their own grammars and stop where the
grammar is complete (tests/engine_contracts.rs:36-60). Beyond those, every constrained draw is compared with the
sampling oracle fed the engine's own logits row and the set of allowed tokens computed here with the `regex`
library's partial matching on the tokens' text - so both the matcher and the place of the mask in the chain
(after bias and penalties, before top_k) are checked from outside."""
import json
from pathlib import Path

import numpy as np
import pytest
import regex

import oracle
from retrograd_amd import engine as E
from retrograd_amd import scheduler as S
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

GOLDEN = json.loads((Path(__file__).resolve().parent / "golden" / "bpe_reference_ids.json").read_text())
KIND = next(k for k in GOLDEN["kinds"] if k["pre"] == "gpt-2")
N_VOCAB = len(KIND["tokens"])
EOS = 1


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    """A small model whose vocabulary is the byte-level one of tests/golden/bpe_reference_ids.json: every byte is a
    token, so every text can be spelled, in many ways."""
    vocab = {"model": "gpt2", "pre": "gpt-2", "tokens": KIND["tokens"], "merges": KIND["merges"],
             "types": [3 if i in KIND["control"] else 1 for i in range(N_VOCAB)], "bos": 0, "eos": EOS}
    shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512,
                         n_vocab=N_VOCAB, name="llama-q4k-grammar")
    p = tmp_path_factory.mktemp("grammar") / "m.gguf"
    synth.write_model(p, shape, seed=77, device="cpu", std=0.2, vocab=vocab)
    return p


def _engine(path):
    return E.Engine(path, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=64, n_ubatch=64))


def test_the_reference_scenario_invalid_forced_and_released(model_path):
    eng = _engine(model_path)
    prompt = eng.tokenize("Hello")
    out = E.StepOutput(1, 4)
    base = dict(temperature=1.0, top_p=1e-6, max_new_tokens=1, seed=17)
    with pytest.raises(E.InvalidArgument, match="invalid GBNF"):
        eng.step([E.StepRow(70, 0, prompt, 0, sample=True, sampling=E.SamplingParamsV2(grammar="root ::= missing", **base),
                            n_top_logprobs=4, want_logprob=True)], out)
    assert eng.seq_pos(0) == (-1, -1)                    # an invalid grammar must not decode a prompt
    eng.step([E.StepRow(70, 0, prompt, 0, sample=True, sampling=E.SamplingParamsV2(**base), n_top_logprobs=4,
                        want_logprob=True)], out)
    first = out.row(0)
    assert first.sampled_logprob == 0.0
    forced = (first.token + 1) % N_VOCAB
    params = dict(base, top_p=1.0)
    eng.step([E.StepRow(70, 0, [first.token], len(prompt), sample=True, want_logprob=True,
                        sampling=E.SamplingParamsV2(grammar="root ::= <[%d]>" % forced, **params))], out)
    assert out.row(0).token == forced and out.row(0).sampled_logprob == 0.0 and not out.row(0).forced
    # the grammar is complete now: a further constrained row would only take an end-of-generation token
    eng.step([E.StepRow(70, 0, [forced], len(prompt) + 1, sample=True,
                        sampling=E.SamplingParamsV2(top_k=1, logit_bias=[(first.token, 100.0)], **params))], out)
    assert out.row(0).token == first.token               # removing the grammar restores unconstrained sampling
    eng.request_free(70)
    eng.close()


def _texts(eng):
    return [eng.detokenize_bytes([t], unparse_special=True) for t in range(N_VOCAB)]


CASES = [
    ('root ::= "Hello" " world"? [0-9]{1,3} ("!" | "?")', rb'Hello( world)?[0-9]{1,3}(!|\?)'),
    ('root ::= ("the " | "The ") word (" " word)* "."\nword ::= [a-z]+', rb'(the |The )[a-z]+( [a-z]+)*\.'),
    ('root ::= "{" ws "\\"k\\"" ws ":" ws [0-9]+ ws "}"\nws ::= [ \\n]*', rb'\{[ \n]*"k"[ \n]*:[ \n]*[0-9]+[ \n]*\}'),
]


@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("top_k", [0, 5])
def test_constrained_draws_equal_the_oracles_on_the_allowed_set(model_path, case, top_k):
    gbnf, pattern = CASES[case]
    rx = regex.compile(pattern, regex.DOTALL)
    eng = _engine(model_path)
    texts = _texts(eng)
    out = E.StepOutput(1, 3)
    for seed in (1, 2, 3):
        # a mild bias towards ending keeps the walks short; it also shows the mask comes after the bias
        params = E.SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=top_k, max_new_tokens=1, seed=seed, grammar=gbnf,
                                    logit_bias=[(EOS, 3.0)], repeat_penalty=1.1)
        rng, history, prefix = oracle.Rng(seed), [], b""
        tokens, pos = eng.tokenize("attention is"), 0
        for step in range(40):
            print("case", case, "top_k", top_k, "seed", seed, "step", step, flush=True)
            eng.step([E.StepRow(seed, 0, tokens, pos, sample=True, sampling=params, n_top_logprobs=3, want_logprob=True)], out)
            logits = eng.debug_logits()[0]
            allowed = np.zeros(N_VOCAB, np.uint8)
            for t in range(N_VOCAB):
                if t == EOS:
                    allowed[t] = rx.fullmatch(prefix) is not None
                elif texts[t]:
                    allowed[t] = rx.fullmatch(prefix + texts[t], partial=True) is not None
            assert allowed.any()
            tok, lp, slp, ids, lps = oracle.sample_v2(logits, rng, temperature=1.0, top_p=1.0, top_k=top_k, repeat_penalty=1.1,
                                                      bias_ids=[EOS], bias_values=[3.0], history=history, k=3, allowed=allowed)
            got = out.row(0)
            assert got.token == tok, (step, prefix, got.token, tok)
            assert allowed[got.token]
            assert got.sampled_logprob == np.float32(slp)
            top_ids, top_lps = out.top(0)
            assert list(top_ids) == list(ids), (step, prefix, top_ids, ids)
            assert all(np.float32(a) == np.float32(b) for a, b in zip(top_lps, lps)), (top_lps, lps)
            history.append(tok)
            pos += len(tokens)
            tokens = [tok]
            if tok == EOS:
                break
            prefix += texts[tok]
        if tok == EOS:
            assert rx.fullmatch(prefix), prefix
        else:                                                 # the open-ended grammars need not end within forty steps
            assert case != 0 and rx.fullmatch(prefix, partial=True), prefix
        eng.seq_rm(0, -1, -1)
        eng.request_free(seed)
    eng.close()


def test_two_rows_of_one_step_keep_their_own_grammars(model_path):
    """tests/engine_contracts.rs:36-60: `root ::= "yes"` and `root ::= "no"` side by side; each text comes out whole
    and the next token can only end the generation. Here through the scheduler over the engine, which hands the
    grammar text of a request to the step as a handle of its own."""
    eng = _engine(model_path)
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=64, queue_capacity=8, event_capacity=64,
                                                           slow_client_timeout=1.0, prefix_cache=False))
    sched.initialize()
    prompt = eng.tokenize("Answer:")
    reqs = [S.Request.single(prompt, E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=8, seed=7,
                                                        grammar='root ::= "%s"' % answer)) for answer in ("yes", "no")]
    outcomes = S.run_requests(sched, reqs)
    for o, answer in zip(outcomes, ("yes", "no")):
        assert o.error is None
        (c,) = o.completions
        assert c.text == answer and c.finish == "Eog" and len(c.tokens) <= 8, (c.text, c.finish)
    # the built-in JSON grammar: whatever the model prefers, the text is a JSON object
    handle = eng._lib.retro_grammar_json_object()
    assert handle
    import ctypes as C
    gbnf = C.string_at(eng._lib.retro_grammar_gbnf(handle)).decode()
    eng._lib.retro_grammar_free(handle)
    (o,) = S.run_requests(sched, [S.Request.single(prompt, E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=200, seed=3,
                                                                              grammar=gbnf, logit_bias=[(EOS, 6.0)]))])
    (c,) = o.completions
    if c.finish == "Eog":
        assert isinstance(json.loads(c.text), dict), c.text
    else:                                                # the budget ran out inside the object: still a prefix of one
        assert c.text.startswith("{")
    # a grammar made from a JSON schema: the text fits the schema (tests/judge_local.rs:82-130 asks the same)
    schema = {"type": "object", "properties": {"verdict": {"enum": ["pass", "fail"]}, "score": {"type": "integer"},
                                               "notes": {"type": "array", "items": {"type": "string", "maxLength": 6}, "maxItems": 2}},
              "required": ["verdict", "score"]}
    handle = eng._lib.retro_grammar_from_json_schema(json.dumps(schema).encode())
    assert handle, E.last_error()
    gbnf = C.string_at(eng._lib.retro_grammar_gbnf(handle)).decode()
    eng._lib.retro_grammar_free(handle)
    assert not eng._lib.retro_grammar_from_json_schema(b'{"type": "string", "pattern": "a+"}') and "'pattern'" in E.last_error()
    (o,) = S.run_requests(sched, [S.Request.single(prompt, E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=120, seed=5,
                                                                              grammar=gbnf, logit_bias=[(EOS, 4.0)]))])
    (c,) = o.completions
    assert c.finish == "Eog", (c.finish, c.text)
    doc = json.loads(c.text)
    assert list(doc)[:2] == ["verdict", "score"] and doc["verdict"] in ("pass", "fail") and isinstance(doc["score"], int)
    assert all(isinstance(n, str) and len(n) <= 6 for n in doc.get("notes", [])) and len(doc.get("notes", [])) <= 2
    sched.close()


# ---- the v2 continuous generator (retro_trainer_generate_continuous_batch_v2, reference retro_gen_core.cpp:2051-2254)

def _trainer(path, n_seq=4):
    from retrograd_amd import trainer as T
    return T.Trainer(path, T.TrainConfig(n_ctx=96, n_batch=16, generation_concurrency=n_seq))


def test_the_v2_generator_keeps_each_rows_grammar(model_path):
    """tests/engine_contracts.rs:36-60 as written: `root ::= "yes"` and `root ::= "no"` in one call; every row's text
    is its grammar's sentence, within its budget, nothing forced; a zero budget is an error."""
    tr = _trainer(model_path)
    prompt = tr.tokenize("Answer:")
    params = lambda answer, n=8: E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=n, seed=7, grammar='root ::= "%s"' % answer)
    rows = tr.generate_continuous_v2([(prompt, params("yes")), (prompt, params("no"))])
    for (tokens, logprobs, forced), expected in zip(rows, ("yes", "no")):
        assert tr.detokenize_bytes(tokens).decode() == expected          # the closing end-of-generation token has no text
        assert tokens[-1] == EOS and len(tokens) <= 8 and len(forced) == len(tokens) and not any(forced)
        assert len(logprobs) == len(tokens) and all(lp <= 0 for lp in logprobs)
    with pytest.raises(E.EngineError):
        tr.generate_continuous_v2([(prompt, params("yes", 0))], n_out_max=4)
    with pytest.raises(E.EngineError, match="invalid GBNF"):
        tr.generate_continuous_v2([(prompt, E.SamplingParamsV2(max_new_tokens=4, grammar="root ::= missing"))])
    assert tr.seq_pos(0) == (-1, -1) or tr.generation_stats()["calls"] >= 1
    tr.close()


def test_a_v2_step_loop_in_canonical_order_reproduces_the_v2_generator_bit_for_bit(model_path, monkeypatch):
    """The relation the reference tests for the v1 generator (tests/engine_runtime.rs:676-724), for the v2 one: the
    canonical order sees the prompts only (the rows' sampling parameters are not part of it), equal prompts are
    decoded once and copied, every row draws from its own generator, history and grammar."""
    monkeypatch.setenv("RETRO_GENERATION_PREFIX_CACHE", "0")
    tr = _trainer(model_path)
    a, b = tr.tokenize("attention is all"), tr.tokenize("the quick brown fox jumps")
    sp = [E.SamplingParamsV2(temperature=0.9, top_p=0.95, top_k=40, max_new_tokens=7, seed=11, repeat_penalty=1.2, penalty_window=4),
          E.SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=0, max_new_tokens=6, seed=12, min_p=0.02, logit_bias=[(5, 1.5)]),
          E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=9, seed=13, grammar='root ::= [a-z ]+ "."', logit_bias=[(EOS, 2.0)]),
          E.SamplingParamsV2(temperature=1.3, top_p=0.8, top_k=5, max_new_tokens=5, seed=14)]
    wave = [(b, sp[0]), (a, sp[1]), (b, sp[2]), (a, sp[3])]
    reference = tr.generate_continuous_v2(wave, 9)

    order = sorted(range(len(wave)), key=lambda i: (len(wave[i][0]), list(wave[i][0]), i))
    slot_of = {seq: slot for slot, seq in enumerate(order)}
    for slot in range(len(order)):
        tr.seq_rm(slot)
    out = E.StepOutput()
    nxt, tokens, lps = {}, {s: [] for s in order}, {s: [] for s in order}

    def row(seq, toks, pos0, sample):
        return E.StepRow(100 + seq, slot_of[seq], toks, pos0, sample=sample, sampling=wave[seq][1])
    g = 0
    while g < len(order):
        leader = order[g]
        prompt = list(wave[leader][0])
        e = g + 1
        while e < len(order) and list(wave[order[e]][0]) == prompt:
            e += 1
        members = order[g:e]
        assert len(members) == 2
        for at in range(0, len(prompt) - 1, 16):
            tr.step([row(leader, prompt[at:min(at + 16, len(prompt) - 1)], at, False)], out)
        for m in members[1:]:
            tr.seq_cp(slot_of[leader], slot_of[m])
        tr.step([row(m, [prompt[-1]], len(prompt) - 1, True) for m in members], out)
        for i, m in enumerate(members):
            nxt[m] = out.row(i)
        g = e
    live = set(order)
    while live:
        active = []
        for s in order:
            if s not in live:
                continue
            tokens[s].append(nxt[s].token)
            lps[s].append(np.float32(nxt[s].logprob))
            if nxt[s].token == EOS or len(tokens[s]) == wave[s][1].max_new_tokens:
                live.discard(s)
            else:
                active.append(s)
        if not active:
            break
        tr.step([row(s, [tokens[s][-1]], len(wave[s][0]) + len(tokens[s]) - 1, True) for s in active], out)
        for i, s in enumerate(active):
            nxt[s] = out.row(i)
    for s in order:
        tr.request_free(100 + s)
    for s, (toks, logprobs, _) in enumerate(reference):
        assert toks == tokens[s], (s, toks, tokens[s])
        assert np.array_equal(np.asarray(logprobs, np.float32).view(np.uint32), np.array(lps[s], np.float32).view(np.uint32))
    text = tr.detokenize_bytes([t for t in reference[2][0] if t != EOS]).decode()
    assert regex.fullmatch(r"[a-z ]+\.?", text), text
    tr.close()
