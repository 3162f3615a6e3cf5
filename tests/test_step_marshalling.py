"""Engine.step fills the FFI rows column by column through a numpy view of the ctypes array: every field of
every row must be what a field-by-field assignment gives, the token pointers must reach the rows' tokens, and the
caller-side errors must come in the reference's order (StepRow::to_ffi_v2 / step_with, reference step.rs:150-203,
412-505). No GPU: the C call is replaced by a recorder."""
import ctypes as C
import types

import numpy as np
import pytest

from retrograd_amd import engine as E


class _Recorder:
    """Stands in for the library: keeps a deep copy of what retro_engine_step_v2 was handed."""

    def __init__(self):
        self.rows = None

    def retro_engine_step_v2(self, handle, ffi_rows, n, out_rows, top_ids, top_lps, stride):
        got = []
        for i in range(n):
            f = ffi_rows[i]
            s = f.sampling
            got.append(dict(
                struct_size=f.struct_size, request=f.request, slot=f.slot, tokens=[f.tokens[j] for j in range(f.n)],
                n=f.n, pos0=f.pos0, sample=bool(f.sample), n_top_logprobs=f.n_top_logprobs, want_logprob=f.want_logprob,
                adapter=f.adapter, s_struct_size=s.struct_size, temperature=s.temperature, top_p=s.top_p,
                max_new_tokens=s.max_new_tokens, seed=s.seed, top_k=s.top_k, min_p=s.min_p, repeat_penalty=s.repeat_penalty,
                frequency_penalty=s.frequency_penalty, presence_penalty=s.presence_penalty, penalty_window=s.penalty_window,
                bias=[(s.logit_bias_ids[j], s.logit_bias_values[j]) for j in range(s.n_logit_bias)],
                bias_null=not bool(s.logit_bias_ids) and not bool(s.logit_bias_values), grammar=s.grammar))
        self.rows = got
        self.stride = stride
        return 0


def _engine():
    rec = _Recorder()
    eng = types.SimpleNamespace(_lib=rec, _h=None)
    eng._fill_sampling_v2 = types.MethodType(E.Engine._fill_sampling_v2, eng)
    eng._check_rows = E.Engine._check_rows
    eng.step = types.MethodType(E.Engine.step, eng)
    return eng, rec


def _f32(x):
    return float(np.float32(x))


def _expect(r):
    s = r.sampling
    return dict(
        struct_size=C.sizeof(E.CStepRowV2), request=r.request, slot=r.slot, tokens=[int(t) for t in r.tokens], n=len(r.tokens),
        pos0=r.pos0, sample=bool(r.sample), n_top_logprobs=r.n_top_logprobs, want_logprob=1 if r.want_logprob else 0,
        adapter=r.adapter.value, s_struct_size=C.sizeof(E.CSamplingParamsV2), temperature=_f32(s.temperature), top_p=_f32(s.top_p),
        max_new_tokens=s.max_new_tokens, seed=s.seed & 0xFFFFFFFF, top_k=s.top_k, min_p=_f32(s.min_p),
        repeat_penalty=_f32(s.repeat_penalty), frequency_penalty=_f32(s.frequency_penalty), presence_penalty=_f32(s.presence_penalty),
        penalty_window=s.penalty_window, bias=[(int(a), _f32(b)) for a, b in s.logit_bias], bias_null=not s.logit_bias, grammar=None)


def test_every_field_of_every_row_reaches_the_c_call():
    rng = np.random.default_rng(5)
    eng, rec = _engine()
    out = E.StepOutput()
    for trial in range(20):
        n = int(rng.integers(1, 70))
        shared = E.SamplingParamsV2(temperature=0.7, top_k=40, seed=2 ** 33 + 5)
        rows = []
        for i in range(n):
            if trial % 3 == 0:
                sp = shared
            else:
                sp = E.SamplingParamsV2(
                    temperature=float(rng.uniform(0.1, 2)), top_p=float(rng.uniform(0.1, 1)), max_new_tokens=int(rng.integers(1, 1000)),
                    seed=int(rng.integers(0, 2 ** 40)), top_k=int(rng.integers(0, 100)), min_p=float(rng.uniform(0, 0.5)),
                    repeat_penalty=float(rng.uniform(0.5, 2)), frequency_penalty=float(rng.uniform(-1, 1)),
                    presence_penalty=float(rng.uniform(-1, 1)), penalty_window=int(rng.integers(0, 512)),
                    logit_bias=[(int(rng.integers(0, 1000)), float(rng.normal())) for _ in range(int(rng.integers(0, 4)))] if i % 5 == 0 else ())
            kind = int(rng.integers(0, 3))
            if trial % 2 == 0 or kind == 0:
                toks = [int(rng.integers(0, 50000))]
            elif kind == 1:
                toks = rng.integers(0, 50000, int(rng.integers(1, 40))).astype(np.int32)
            else:
                toks = [int(t) for t in rng.integers(0, 50000, int(rng.integers(1, 9)))]
            rows.append(E.StepRow(request=i if i % 7 else -1 - i, slot=int(rng.integers(0, 64)), tokens=toks,
                                  pos0=int(rng.integers(0, 1 << 20)), sample=bool(i % 7) and bool(rng.integers(0, 2)), sampling=sp,
                                  n_top_logprobs=int(rng.integers(0, 5)), want_logprob=bool(rng.integers(0, 2)),
                                  adapter=E.RowAdapter(int(rng.integers(-1, 4)))))
        eng.step(rows, out)
        assert rec.stride == max(r.n_top_logprobs for r in rows)
        assert len(rec.rows) == n
        for got, r in zip(rec.rows, rows):
            assert got == _expect(r)


def test_rows_left_from_a_larger_step_do_not_leak_into_a_smaller_one():
    eng, rec = _engine()
    out = E.StepOutput()
    biased = E.SamplingParamsV2(logit_bias=[(3, 1.5)])
    eng.step([E.StepRow(i, i, [i], 0, sample=True, sampling=biased) for i in range(8)], out)
    assert all(g["bias"] == [(3, 1.5)] for g in rec.rows)
    plain = [E.StepRow(i, i, [7, 8], 5, sample=True) for i in range(3)]
    eng.step(plain, out)
    assert [g == _expect(r) for g, r in zip(rec.rows, plain)] == [True] * 3


def test_integers_wider_than_their_field_wrap_as_a_ctypes_assignment_does():
    eng, rec = _engine()
    out = E.StepOutput()
    rows = [E.StepRow((1 << 40) + i, i, [1], 0, sample=True, sampling=E.SamplingParamsV2(max_new_tokens=(1 << 32) + 7, top_k=-1))
            for i in range(3)]
    eng.step(rows, out)
    assert [g["request"] for g in rec.rows] == [0, 1, 2]
    assert [g["max_new_tokens"] for g in rec.rows] == [7, 7, 7]
    assert [g["top_k"] for g in rec.rows] == [-1, -1, -1]
    shared = E.SamplingParamsV2(max_new_tokens=(1 << 32) + 9)
    eng.step([E.StepRow((1 << 40) + i, i, [1], 0, sample=True, sampling=shared) for i in range(3)], out)
    assert [g["max_new_tokens"] for g in rec.rows] == [9, 9, 9]


def test_caller_side_errors_come_in_row_order():
    eng, _ = _engine()
    out = E.StepOutput()
    ok = E.StepRow(0, 0, [1], 0, sample=True)
    with pytest.raises(E.InvalidArgument, match="at least one token"):
        eng.step([ok, E.StepRow(1, 1, [], 0), E.StepRow(2, 2, [1], -1)], out)
    with pytest.raises(E.InvalidArgument, match="pos0 must be >= 0"):
        eng.step([ok, E.StepRow(2, 2, [1], -1), E.StepRow(1, 1, [], 0)], out)
    with pytest.raises(E.EngineError, match="overflows i32"):
        eng.step([E.StepRow(1, 1, [1, 2], 2 ** 31 - 2)], out)
    with pytest.raises(E.InvalidArgument, match="request id >= 0"):
        eng.step([E.StepRow(-1, 1, [1], 0, sample=True)], out)
    with pytest.raises(E.InvalidArgument, match="at most 4096"):
        eng.step([E.StepRow(1, 1, [1], 0, sampling=E.SamplingParamsV2(logit_bias=[(1, 0.0)] * 4097))], out)
    with pytest.raises(E.InvalidArgument, match="appears twice"):
        eng.step([ok, E.StepRow(5, 1, [1], 0), E.StepRow(5, 2, [1], 0)], out)
    eng.step([E.StepRow(-1, 1, [1], 0), E.StepRow(-1, 2, [1], 0)], out)        # rows without a request may repeat -1
    eng.step([], out)
