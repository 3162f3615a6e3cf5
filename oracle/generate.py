"""TEST INFRASTRUCTURE - CPU oracle of the batched generators, never imported by
the product.

A Python restatement of retro_engine_generate_batch and
retro_engine_generate_continuous_batch, written from the reference's C++
(crates/retrograd-ffi/runtime/src/retro_gen_core.cpp) and independent of
retrograd_amd/csrc/generate.cpp:

  * canonical order            retro_gen_core.cpp:333-358
  * slot placement, eviction   retro_gen_core.cpp:430-546
  * what a slot remembers      retro_gen_core.cpp:557-582
  * grouped chunked prefill    retro_gen_core.cpp:585-705
  * generate_batch             retro_gen_core.cpp:1696-1876
  * generate_continuous_batch  retro_gen_core.cpp:1878-2049
  * v1 sampling and logprob    retro_gen_core.cpp:103-129, 1830-1836 (oracle.sample_v1)

It runs over any backend with `decode(rows) -> logits of the rows that ask`,
`seq_rm` and `seq_cp`: oracle.Context (the CPU forward pass) or a synthetic one
whose logits are a closed form of the row's history (tests/test_generators.py).
Pinned by the reference's own scenarios (tests/engine_runtime.rs:294-306,
362-404, 676-724; tests/infer_runtime.rs:90-197) and by hand-derived counters.
"""

from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

import numpy as np

import oracle

Sampling = Tuple[float, float, int, int]          # temperature, top_p, max_new_tokens, seed


class GenerationError(RuntimeError):
    pass


@dataclass
class Stats:
    calls: int = 0
    sequences: int = 0
    prompt_tokens: int = 0
    prefilled_tokens: int = 0
    reused_tokens: int = 0
    hits: int = 0
    evictions: int = 0

    def as_dict(self) -> dict:
        return dict(self.__dict__)


def canonical_order(sequences: Sequence[Tuple[Sequence[int], Sampling]]) -> List[int]:
    def key(i):
        prompt, (temperature, top_p, max_new, seed) = sequences[i]
        return (len(prompt), tuple(int(t) for t in prompt), seed & 0xFFFFFFFF, max_new, np.float32(temperature), np.float32(top_p))
    return sorted(range(len(sequences)), key=key)       # sorted() is stable, as std::stable_sort


def _validate_sampling(p: Sampling) -> None:
    temperature, top_p, max_new, _ = p
    if not (temperature > 0.0) or not np.isfinite(temperature):
        raise GenerationError("sampling temperature must be finite and greater than zero")
    if not (0.0 < top_p <= 1.0):
        raise GenerationError("sampling top_p must be in (0, 1]")
    if max_new == 0:
        raise GenerationError("sampling max_new_tokens must be greater than zero")


@dataclass
class Generator:
    backend: object
    n_seq_max: int
    n_batch: int
    n_ctx: int               # cells of the whole pool
    n_ctx_seq: int           # positions one sequence may hold
    n_vocab: int
    eog: Sequence[int] = ()
    slots: List[List[int]] = field(default_factory=list)      # resident tokens per slot
    used_at: List[int] = field(default_factory=list)
    clock: int = 0
    stats: Stats = field(default_factory=Stats)
    launches: List[List[Tuple[int, int, int, bool]]] = field(default_factory=list)   # (slot, pos0, n, logits) per decode

    # ---- plumbing -------------------------------------------------------------------
    def _decode(self, rows):
        self.launches.append([(slot, pos0, len(tokens), bool(want)) for slot, pos0, tokens, want in rows])
        return self.backend.decode(rows)

    def forget(self) -> None:
        self.slots = [[] for _ in self.slots]
        self.used_at = [0 for _ in self.used_at]

    def clear_generation_memory(self) -> None:
        for slot in range(self.n_seq_max):
            self.backend.seq_rm(slot, -1, -1)
        self.forget()

    def _validate_tokens(self, tokens) -> None:
        for i, t in enumerate(tokens):
            if t < 0 or t >= self.n_vocab:
                raise GenerationError("token %d at index %d is outside the vocabulary of size %d" % (t, i, self.n_vocab))

    def _sample(self, logits, p: Sampling, rng):
        temperature, top_p, _, _ = p
        token, logprob, _, _ = oracle.sample_v1(logits, temperature, top_p, rng)
        return token, np.float32(logprob)

    # ---- generate_batch ---------------------------------------------------------------
    def generate_batch(self, prompt: Sequence[int], sampling: Sequence[Sampling], n_out_max: int):
        n = len(sampling)
        if len(prompt) == 0:
            raise GenerationError("prompt tokens are required")
        if n == 0 or n_out_max == 0:
            raise GenerationError("sampling params and output buffers are required")
        if n > self.n_seq_max:
            raise GenerationError("generation batch has %d sequences but the context supports %d" % (n, self.n_seq_max))
        if n > self.n_batch:
            raise GenerationError("generation batch exceeds the configured batch capacity")
        for p in sampling:
            _validate_sampling(p)
        self._validate_tokens(prompt)
        n_prompt = len(prompt)
        if n_prompt >= self.n_ctx_seq:
            raise GenerationError("prompt of %d tokens leaves no room to generate in context %d" % (n_prompt, self.n_ctx_seq))
        self.clear_generation_memory()
        # the prompt is decoded once, in slot 0, n_batch positions per launch; only the last row asks for logits
        logits = None
        for at in range(0, n_prompt, self.n_batch):
            chunk = list(prompt[at:at + self.n_batch])
            last = at + len(chunk) == n_prompt
            got = self._decode([(0, at, chunk, last)])
            if last:
                logits = got[0]
        for member in range(1, n):
            self.backend.seq_cp(0, member, -1, -1)
        rngs = [oracle.Rng(p[3]) for p in sampling]
        row_logits = [logits] * n
        limits = [min(n_out_max, p[2], self.n_ctx_seq - n_prompt) for p in sampling]
        out = [([], []) for _ in range(n)]
        live = [True] * n
        while any(live):
            decoded = []
            for i in range(n):
                if not live[i]:
                    continue
                token, lp = self._sample(row_logits[i], sampling[i], rngs[i])
                out[i][0].append(token)
                out[i][1].append(lp)
                if token in self.eog or len(out[i][0]) == limits[i]:
                    live[i] = False
                else:
                    decoded.append(i)
            if not decoded:
                break
            got = self._decode([(i, n_prompt + len(out[i][0]) - 1, [out[i][0][-1]], True) for i in decoded])
            for r, i in enumerate(decoded):
                row_logits[i] = got[r]
        self.clear_generation_memory()
        return [(toks, np.array(lps, np.float32)) for toks, lps in out]

    # ---- generate_continuous_batch ----------------------------------------------------
    @staticmethod
    def _resident_prefix(resident: List[int], prompt: Sequence[int]) -> int:
        if not resident or len(resident) >= len(prompt):
            return 0
        return len(resident) if list(prompt[:len(resident)]) == resident else 0

    def _place(self, sequences, order, n_out_max, cache: bool):
        n = len(sequences)
        if not cache:
            return list(range(n)), [0] * n
        if len(self.slots) < self.n_seq_max:
            self.slots += [[] for _ in range(self.n_seq_max - len(self.slots))]
            self.used_at += [0] * (self.n_seq_max - len(self.used_at))
        slot_of, reuse_of = [0] * n, [0] * n
        claimed = [False] * self.n_seq_max
        for seq in order:
            prompt, _ = sequences[seq]
            best_slot, best_reuse = self.n_seq_max, 0
            for slot in range(self.n_seq_max):
                if claimed[slot]:
                    continue
                reuse = self._resident_prefix(self.slots[slot], prompt)
                if best_slot == self.n_seq_max or reuse > best_reuse:
                    best_slot, best_reuse = slot, reuse
                    continue
                if reuse == best_reuse and reuse == 0 and self.used_at[slot] < self.used_at[best_slot]:
                    best_slot = slot
            claimed[best_slot] = True
            slot_of[seq], reuse_of[seq] = best_slot, best_reuse
            if best_reuse == 0:
                if self.slots[best_slot]:
                    self.stats.evictions += 1
                self.backend.seq_rm(best_slot, -1, -1)
                self.slots[best_slot] = []
            else:
                self.stats.hits += 1
            self.stats.sequences += 1
            self.stats.prompt_tokens += len(prompt)
            self.stats.reused_tokens += best_reuse
        remaining = self.n_ctx
        for prompt, p in sequences:
            emitted = min(n_out_max, p[2], self.n_ctx_seq - len(prompt))
            remaining -= min(remaining, len(prompt) + emitted - 1)
        dormant = sum(len(self.slots[s]) for s in range(self.n_seq_max) if not claimed[s])
        while dormant > remaining:
            candidates = [s for s in range(self.n_seq_max) if not claimed[s] and self.slots[s]]
            if not candidates:
                break
            oldest = min(candidates, key=lambda s: (self.used_at[s], s))
            self.backend.seq_rm(oldest, -1, -1)
            dormant -= len(self.slots[oldest])
            self.slots[oldest] = []
            self.used_at[oldest] = 0
            self.stats.evictions += 1
        return slot_of, reuse_of

    def _prefill(self, sequences, order, slot_of, reuse_of):
        """Chunked, grouped prefill; returns the terminal logits per sequence."""
        terminal_logits = [None] * len(sequences)
        pending, wanted = [], []          # rows of the pending launch; sequences waiting on its logits

        def flush():
            if not pending:
                return
            # one row per pushed position, merged into runs of one slot
            rows = []
            for slot, pos, token, want in pending:
                if rows and rows[-1][0] == slot and rows[-1][1] + len(rows[-1][2]) == pos and not rows[-1][3]:
                    rows[-1] = (slot, rows[-1][1], rows[-1][2] + [token], want)
                else:
                    rows.append((slot, pos, [token], want))
            got = self._decode(rows)
            for k, seq in enumerate(wanted):
                terminal_logits[seq] = got[k]
            pending.clear()
            wanted.clear()

        def push(seq, pos, token, want):
            if len(pending) == self.n_batch:
                flush()
            pending.append((slot_of[seq], pos, token, want))
            if want:
                wanted.append(seq)
            self.stats.prefilled_tokens += 1

        g = 0
        while g < len(order):
            leader = order[g]
            prompt, _ = sequences[leader]
            reuse = reuse_of[leader]
            e = g + 1
            if reuse == 0:
                while e < len(order) and reuse_of[order[e]] == 0 and list(sequences[order[e]][0]) == list(prompt):
                    e += 1
            for pos in range(reuse, len(prompt) - 1):
                push(leader, pos, prompt[pos], False)
            if e > g + 1:
                flush()
                for m in range(g + 1, e):
                    self.backend.seq_cp(slot_of[leader], slot_of[order[m]], -1, -1)
            for m in range(g, e):
                push(order[m], len(prompt) - 1, prompt[-1], True)
            flush()
            g = e
        return terminal_logits

    def generate_continuous_batch(self, sequences: Sequence[Tuple[Sequence[int], Sampling]], n_out_max: int):
        n = len(sequences)
        if n == 0 or n_out_max == 0:
            raise GenerationError("continuous generation inputs and output buffers are required")
        if n > self.n_seq_max or n > self.n_batch:
            raise GenerationError("continuous generation batch exceeds the configured sequence or batch capacity")
        for prompt, p in sequences:
            if len(prompt) == 0 or len(prompt) >= self.n_ctx_seq:
                raise GenerationError("invalid continuous generation prompt")
            _validate_sampling(p)
            self._validate_tokens(prompt)
        value = os.environ.get("RETRO_GENERATION_PREFIX_CACHE")
        cache = not (value in ("0", "false"))
        if not cache:
            self.clear_generation_memory()
        self.stats.calls += 1
        order = canonical_order(sequences)
        slot_of, reuse_of = self._place(sequences, order, n_out_max, cache)
        row_logits = self._prefill(sequences, order, slot_of, reuse_of)
        rngs = [oracle.Rng(p[3]) for _, p in sequences]
        limits = [min(n_out_max, p[2], self.n_ctx_seq - len(prompt)) for prompt, p in sequences]
        out = [([], []) for _ in range(n)]
        live = [True] * n
        while any(live):
            active = []
            for seq in order:
                if not live[seq]:
                    continue
                token, lp = self._sample(row_logits[seq], sequences[seq][1], rngs[seq])
                out[seq][0].append(token)
                out[seq][1].append(lp)
                if token in self.eog or len(out[seq][0]) == limits[seq]:
                    live[seq] = False
                else:
                    active.append(seq)
            if not active:
                break
            got = self._decode([(slot_of[s], len(sequences[s][0]) + len(out[s][0]) - 1, [out[s][0][-1]], True) for s in active])
            for r, s in enumerate(active):
                row_logits[s] = got[r]
        if cache:
            self.clock += 1
            for s in range(n):
                decoded = max(len(out[s][0]) - 1, 0)
                self.slots[slot_of[s]] = [int(t) for t in sequences[s][0]] + [int(t) for t in out[s][0][:decoded]]
                self.used_at[slot_of[s]] = self.clock
        else:
            self.clear_generation_memory()
        return [(toks, np.array(lps, np.float32)) for toks, lps in out]


class ContextBackend:
    """oracle.Context as a generator backend."""

    def __init__(self, ctx: "oracle.Context") -> None:
        self.ctx = ctx

    def decode(self, rows):
        return self.ctx.step_rows([(slot, pos0, [int(t) for t in tokens], bool(want)) for slot, pos0, tokens, want in rows])

    def seq_rm(self, slot, p0, p1):
        self.ctx.seq_rm(slot, p0, p1)

    def seq_cp(self, src, dst, p0, p1):
        self.ctx.seq_cp(src, dst, p0, p1)
