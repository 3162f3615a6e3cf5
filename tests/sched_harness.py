"""One interface over the two scheduler implementations, so every policy
scenario runs on both: the product (C++ behind include/retro_scheduler.h) and
the oracle (oracle/scheduler.py)."""

from __future__ import annotations

from typing import List, Optional, Sequence

from oracle import scheduler as O
from retrograd_amd import engine as E
from retrograd_amd import scheduler as S

LOCKSTEP, CONTINUOUS = 0, 1


def pieces(vocab: int) -> List[str]:
    """The piece table the reference's scheduler tests use (tests/fake_backend.rs:15-27)."""
    return ["" if i == 99 else chr(ord("a") + i % 26) for i in range(vocab)]


class Harness:
    """kind: "product" or "oracle". Requests are dicts: prompt, sampling = [(seed, max_new), ...] or full dicts."""

    def __init__(self, kind: str, n_slots: int, n_ctx_seq: int, cells_total: int, vocab: int = 100, eos: int = 99,
                 piece_table: Optional[Sequence] = None, **options):
        self.kind = kind
        table = list(piece_table) if piece_table is not None else pieces(vocab)
        if kind == "product":
            opts = S.SchedulerOptions(**options)
            raw = [p if isinstance(p, bytes) else p.encode("utf-8") for p in table]
            self.s = _product_over_fake(n_slots, n_ctx_seq, cells_total, vocab, eos, raw, opts)
        else:
            self.backend = O.FakeBackend(n_slots, n_ctx_seq, cells_total, vocab, eos,
                                         [p.decode("utf-8", "surrogateescape") if isinstance(p, bytes) else p for p in table])
            if any(isinstance(p, bytes) for p in table):
                self.backend.detokenize_bytes = _bytes_detok(self.backend, table)
            self.s = O.Scheduler(self.backend, O.Options(**options))
        self.s.initialize()

    # -- fake knobs
    def set(self, key: str, value=0):
        if self.kind == "product":
            self.s.fake.set(key, int(value))
        else:
            b = self.backend
            if key == "eog_after":
                b.eog_after = None if value < 0 else value
            elif key == "kv_unified":
                b.kv_unified_flag = bool(value)
            elif key == "recurrent":
                b.recurrent = bool(value)
            elif key == "row_adapters":
                b.row_adapters_enabled = bool(value)
            elif key == "fail_after_steps":
                b.fail_after_steps = value
            elif key == "bump_weights_version":
                b.bump_weights_version()
            else:
                raise KeyError(key)

    def script(self, tokens):
        if self.kind == "product":
            self.s.fake.script(list(tokens))
        else:
            self.backend.script = list(tokens)

    def register_adapter(self, name, path="p"):
        if self.kind == "product":
            self.s.fake.register_adapter(name, path)
        else:
            self.backend.register_adapter(name, path)

    # -- requests
    def submit(self, prompt, sampling, **kw):
        if self.kind == "product":
            samp = [_product_sampling(s) for s in sampling]
            ret = kw.pop("retention", None)
            req = S.Request(list(prompt), samp, retention=S.Retention(*ret) if ret else None, **kw)
            return self.s.submit(req)
        samp = [_oracle_sampling(s) for s in sampling]
        if "stop" in kw:
            kw["stop"] = list(kw["stop"])
        return self.s.submit(O.Request(list(prompt), samp, **kw))

    def drop(self, stream):
        """Dropping the receiving end: buffered events are gone with it."""
        if self.kind == "product":
            stream.close()
        else:
            stream.drop()
            stream.queue.clear()
            stream.dropped = True

    def events(self, stream):
        """Drains the buffered events, normalised."""
        out = []
        if self.kind == "product":
            for e in stream.drain():
                if e.type == "Token":
                    out.append(("T", e.index, e.token, e.text, e.piece, _r(e.logprob), _r(e.sampled_logprob), e.forced,
                                [(t.token, _r(t.logprob), t.piece) for t in e.top_logprobs]))
                elif e.type == "End":
                    out.append(("E", e.index, e.reason, e.text, e.cached_tokens))
                else:
                    out.append(("X", e.error.kind, e.error.message, e.error.needed, e.error.available))
        elif not getattr(stream, "dropped", False):
            for e in stream.drain():
                if e["type"] == "Token":
                    out.append(("T", e["index"], e["token"], e["text"], e["piece"], _r(e["logprob"]),
                                _r(e["sampled_logprob"]), e["forced"],
                                [(t, _r(lp), p) for t, lp, p in e["top_logprobs"]]))
                elif e["type"] == "End":
                    out.append(("E", e["index"], e["reason"], e["text"], e["cached_tokens"]))
                else:
                    err = e["error"]
                    out.append(("X", err.kind, err.message, err.needed, err.available))
        return out

    def closed(self, stream) -> bool:
        if self.kind == "product":
            return stream.poll()[0] == "Closed"
        return getattr(stream, "dropped", False) or stream.closed()

    # -- driver
    def pump(self) -> bool:
        return self.s.pump()

    def run_until_idle(self):
        self.s.run_until_idle()

    def run_requests(self, requests):
        """sync.rs run_requests; requests are (prompt, sampling) pairs. Returns per request
        (completions [(tokens, rounded logprobs, forced, text, finish)], error kind or None)."""
        if self.kind == "product":
            reqs = [S.Request(list(p), [_product_sampling(x) for x in samp]) for p, samp in requests]
            return [([(c.tokens, [_r(v) for v in c.logprobs], c.forced, c.text, c.finish) for c in o.completions],
                     o.error.kind if o.error else None) for o in S.run_requests(self.s, reqs)]
        reqs = [O.Request(list(p), [_oracle_sampling(x) for x in samp]) for p, samp in requests]
        return [([(c["tokens"], [_r(v) for v in c["logprobs"]], c["forced"], c["text"], c["finish"]) for c in o["completions"]],
                 o["error"].kind if o["error"] else None) for o in O.run_requests(self.s, reqs)]

    def lend_slot(self, cells):
        return self.s.lend_slot(cells)

    def seq_pos(self, slot):
        return self.s.fake.seq_pos(slot) if self.kind == "product" else self.backend.seq_pos(slot)

    def cells_used(self):
        return self.s.fake.cells_used if self.kind == "product" else self.backend.cells_used()

    def is_idle(self):
        return self.s.is_idle()

    def queued(self) -> int:
        return self.s.queued_len()

    def live(self) -> int:
        return self.s.live_len()

    def set_mode(self, mode):
        if self.kind == "product":
            self.s.set_mode(mode)
        else:
            self.s.o.mode = mode

    def kv_stats(self) -> dict:
        if self.kind == "product":
            k = self.s.kv_stats()
            return dict(hits=k.hits, misses=k.misses, prefilled_cells=k.prefilled_cells, prompt_cells=k.prompt_cells,
                        evictions=k.evictions, swaps=k.swaps, nodes=k.nodes, resident_slots=k.resident_slots,
                        snapshot_bytes=k.snapshot_bytes)
        return self.s.kv_stats()

    def pin_prefix(self, prefix):
        return self.s.pin_prefix(list(prefix))

    def unpin(self, pin):
        return self.s.unpin(pin)

    def load_adapter(self, name, path="p"):
        self.s.load_adapter(name, path)

    def unload_adapter(self, name):
        self.s.unload_adapter(name)

    # -- fake log
    def log(self) -> dict:
        if self.kind == "product":
            f = self.s.fake
            return dict(steps=f.steps, step_adapters=f.step_adapters, copies=[tuple(c) for c in f.copies],
                        removed=f.removed, request_order=f.request_order, saves=[tuple(s) for s in f.saves],
                        loads=[tuple(s) for s in f.loads], adapter_ops=f.adapter_ops, cells_used=f.cells_used)
        b = self.backend
        return dict(steps=[list(s) for s in b.steps], step_adapters=[list(s) for s in b.step_adapters],
                    copies=list(b.copies), removed=list(b.removed), request_order=list(b.request_order),
                    saves=list(b.saves), loads=list(b.loads), adapter_ops=list(b.adapter_ops),
                    cells_used=b.cells_used())

    @property
    def error_type(self):
        return S.InferError if self.kind == "product" else O.InferError


def _r(x):
    return None if x is None else round(float(x), 5)


def _norm(s):
    if isinstance(s, tuple):
        return dict(seed=s[0], max_new_tokens=s[1])
    return dict(s)


def _product_sampling(s):
    d = _norm(s)
    bias = d.pop("logit_bias", ())
    grammar = d.pop("grammar_gbnf", None)
    return E.SamplingParamsV2(logit_bias=tuple(bias), grammar=grammar, **d)


def _oracle_sampling(s):
    d = _norm(s)
    d["logit_bias"] = tuple(d.get("logit_bias", ()))
    return O.Sampling(**d)


def _bytes_detok(backend, table):
    raw = [p if isinstance(p, bytes) else p.encode("utf-8") for p in table]

    def detok(tokens, unparse_special):
        out = b""
        for t in tokens:
            if t == backend.eos and not unparse_special:
                continue
            out += raw[t] if 0 <= t < len(raw) else ("<%d>" % t).encode()
        return out
    return detok


def _product_over_fake(n_slots, n_ctx_seq, cells_total, vocab, eos, raw_pieces, opts):
    import ctypes as C
    lib = S._lib()
    c_opts = opts.to_c()
    arr = (C.c_char_p * max(len(raw_pieces), 1))(*raw_pieces)
    return S.Scheduler(lib.retro_scheduler_new_fake(n_slots, n_ctx_seq, cells_total, vocab, eos, arr, len(raw_pieces),
                                                    C.byref(c_opts)), fake=True)
