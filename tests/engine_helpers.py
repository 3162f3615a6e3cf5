"""Shared helpers of the GPU step tests: run the same plan through the engine
(C ABI) and through the CPU oracle."""
import numpy as np

import oracle
from retrograd_amd import engine as E


def greedy():
    return E.SamplingParamsV2.greedy()


def run_both(eng, ctx, rows):
    """rows: (request, slot, tokens, pos0, sample). Returns (StepOutput, engine
    logits, oracle logits)."""
    out = E.StepOutput()
    eng.step([E.StepRow(r[0], r[1], r[2], r[3], sample=r[4], sampling=greedy()) for r in rows], out)
    want = ctx.step_rows([(r[1], r[3], r[2], r[4]) for r in rows])
    got = eng.debug_logits()
    return out, got, want


def logit_errors(got, want):
    """max-abs error and mean-abs error relative to the mean-abs logit."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return err.max(), err.mean() / np.abs(want).mean()


def assert_logits_close(got, want, max_abs=2e-2, mean_rel=1e-3):
    assert got.shape == want.shape
    mx, mr = logit_errors(got, want)
    assert mx <= max_abs and mr <= mean_rel, (mx, mr)
