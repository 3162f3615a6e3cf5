"""Host-side mirror of the step scheduler's C ABI (include/retro_scheduler.h).

The names follow the reference's retrograd-infer crate: `Scheduler.submit`,
`pump`, `run_until_idle`, `kv_stats`, `pin_prefix`, `Request`, `Event`,
`EventStream`, `FakeBackend` (crates/retrograd-infer/src/scheduler.rs,
request.rs, fake.rs). The policy itself runs in C++ inside libretro_hip.so;
nothing here decides anything.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

from . import engine as E

LOCKSTEP, CONTINUOUS = 0, 1
EVENT_TOKEN, EVENT_END, EVENT_ERROR = 0, 1, 2
FINISH = {0: "Eog", 1: "Stop", 2: "MaxTokens", 3: "ContextFull", 4: "Cancelled"}
ERROR_KINDS = {1: "InvalidArgument", 2: "Failed", 3: "Overflow", 4: "QueueFull", 5: "KvFull", 6: "Cancelled",
               7: "Backend"}

SCHED_SYMBOLS = [
    "retro_sched_options_default", "retro_scheduler_new", "retro_scheduler_new_trainer", "retro_scheduler_new_fake", "retro_scheduler_lend_slot",
    "retro_scheduler_queue_capacity", "retro_scheduler_free",
    "retro_scheduler_initialize", "retro_scheduler_submit", "retro_scheduler_pump", "retro_scheduler_run_until_idle",
    "retro_scheduler_counts", "retro_scheduler_fail_queued", "retro_scheduler_kv_stats", "retro_scheduler_pin_prefix",
    "retro_scheduler_unpin", "retro_scheduler_load_adapter", "retro_scheduler_unload_adapter",
    "retro_scheduler_set_mode", "retro_sched_last_error_detail", "retro_sched_stream_poll", "retro_sched_stream_free",
    "retro_sched_fake_set", "retro_sched_fake_script", "retro_sched_fake_register_adapter",
    "retro_sched_fake_cells_used", "retro_sched_fake_log", "retro_sched_fake_adapter_ops",
]


class InferError(RuntimeError):
    """crates/retrograd-infer/src/error.rs:8-27; `kind` names the variant."""

    def __init__(self, kind: str, message: str, needed: int = 0, available: int = 0, capacity: int = 0):
        super().__init__("%s: %s" % (kind, message))
        self.kind, self.message = kind, message
        self.needed, self.available, self.capacity = needed, available, capacity


class COptions(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("mode", C.c_int32), ("n_batch", C.c_uint64),
                ("queue_capacity", C.c_uint64), ("event_capacity", C.c_uint64),
                ("slow_client_timeout_ns", C.c_uint64), ("prefix_cache", C.c_uint8), ("min_prefix_len", C.c_uint64),
                ("max_snapshot_bytes", C.c_uint64), ("swap_min_tokens", C.c_uint64), ("max_retained", C.c_uint64),
                ("retain_ttl_ns", C.c_uint64)]


class CRequest(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("prompt", C.POINTER(C.c_int32)), ("n_prompt", C.c_size_t),
                ("sampling", C.POINTER(E.CSamplingParamsV2)), ("n_sampling", C.c_size_t),
                ("grammar_gbnf", C.POINTER(C.c_char_p)), ("stop", C.POINTER(C.c_char_p)), ("n_stop", C.c_size_t),
                ("n_top_logprobs", C.c_uint32), ("logprobs", C.c_uint8), ("adapter", C.c_char_p),
                ("unparse_special", C.c_uint8), ("retention_key", C.c_char_p), ("retention_release", C.c_char_p)]


class CEvent(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("type", C.c_int32), ("index", C.c_uint64), ("token", C.c_int32),
                ("logprob", C.c_float), ("has_sampled_logprob", C.c_uint8), ("sampled_logprob", C.c_float),
                ("forced", C.c_uint8), ("text", C.c_void_p), ("n_text", C.c_size_t), ("piece", C.c_void_p),
                ("n_piece", C.c_size_t), ("n_top", C.c_size_t), ("top_ids", C.POINTER(C.c_int32)),
                ("top_logprobs", C.POINTER(C.c_float)), ("top_pieces", C.POINTER(C.c_void_p)),
                ("top_piece_lens", C.POINTER(C.c_size_t)), ("reason", C.c_int32), ("cached_tokens", C.c_uint64),
                ("error_kind", C.c_int32), ("error_message", C.c_char_p), ("error_needed", C.c_uint64),
                ("error_available", C.c_uint64)]


class CKvStats(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("hits", C.c_uint64), ("misses", C.c_uint64),
                ("prefilled_cells", C.c_uint64), ("prompt_cells", C.c_uint64), ("evictions", C.c_uint64),
                ("swaps", C.c_uint64), ("nodes", C.c_uint64), ("resident_slots", C.c_uint64),
                ("snapshot_bytes", C.c_uint64)]


_bound = False


def _lib() -> C.CDLL:
    global _bound
    lib = E.load_library()
    if not _bound:
        lib.retro_scheduler_new.restype = C.c_void_p
        lib.retro_scheduler_new.argtypes = [C.c_void_p, C.POINTER(COptions)]
        lib.retro_scheduler_lend_slot.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_int32)]
        lib.retro_scheduler_queue_capacity.argtypes = [C.c_void_p, C.POINTER(C.c_size_t)]
        lib.retro_scheduler_new_trainer.restype = C.c_void_p
        lib.retro_scheduler_new_trainer.argtypes = [C.c_void_p, C.POINTER(COptions)]
        lib.retro_scheduler_new_fake.restype = C.c_void_p
        lib.retro_scheduler_new_fake.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32, C.c_int32,
                                                 C.POINTER(C.c_char_p), C.c_size_t, C.POINTER(COptions)]
        lib.retro_scheduler_free.argtypes = [C.c_void_p]
        lib.retro_scheduler_free.restype = None
        lib.retro_sched_options_default.argtypes = [C.POINTER(COptions)]
        lib.retro_sched_options_default.restype = None
        lib.retro_scheduler_initialize.argtypes = [C.c_void_p]
        lib.retro_scheduler_submit.argtypes = [C.c_void_p, C.POINTER(CRequest), C.POINTER(C.c_void_p)]
        lib.retro_scheduler_pump.argtypes = [C.c_void_p, C.POINTER(C.c_uint8)]
        lib.retro_scheduler_run_until_idle.argtypes = [C.c_void_p]
        lib.retro_scheduler_counts.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        lib.retro_scheduler_fail_queued.argtypes = [C.c_void_p]
        lib.retro_scheduler_kv_stats.argtypes = [C.c_void_p, C.POINTER(CKvStats)]
        lib.retro_scheduler_pin_prefix.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.c_size_t, C.POINTER(C.c_uint64)]
        lib.retro_scheduler_unpin.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint8)]
        lib.retro_scheduler_load_adapter.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
        lib.retro_scheduler_unload_adapter.argtypes = [C.c_void_p, C.c_char_p]
        lib.retro_scheduler_set_mode.argtypes = [C.c_void_p, C.c_int32]
        lib.retro_sched_last_error_detail.argtypes = [C.POINTER(C.c_uint64)] * 3
        lib.retro_sched_last_error_detail.restype = None
        lib.retro_sched_stream_poll.argtypes = [C.c_void_p, C.POINTER(CEvent)]
        lib.retro_sched_stream_free.argtypes = [C.c_void_p]
        lib.retro_sched_stream_free.restype = None
        lib.retro_sched_fake_set.argtypes = [C.c_void_p, C.c_char_p, C.c_int64]
        lib.retro_sched_fake_script.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.c_size_t]
        lib.retro_sched_fake_register_adapter.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
        lib.retro_sched_fake_cells_used.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
        lib.retro_sched_fake_log.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64), C.c_size_t,
                                             C.POINTER(C.c_size_t)]
        lib.retro_sched_fake_adapter_ops.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
        _bound = True
    return lib


def _check(status: int) -> None:
    if status == 0:
        return
    lib = _lib()
    n, a, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
    lib.retro_sched_last_error_detail(C.byref(n), C.byref(a), C.byref(c))
    raise InferError(ERROR_KINDS.get(-status, "Failed"), E.last_error(), n.value, a.value, c.value)


@dataclass
class SchedulerOptions:
    """crates/retrograd-infer/src/scheduler.rs:86-135 (same defaults)."""
    mode: int = LOCKSTEP
    n_batch: int = 512
    queue_capacity: int = 64
    event_capacity: int = 64
    slow_client_timeout: float = 5.0
    prefix_cache: bool = True
    min_prefix_len: int = 8
    max_snapshot_bytes: int = 256 << 20
    swap_min_tokens: int = 256
    max_retained: int = 8
    retain_ttl: float = 300.0

    def to_c(self) -> COptions:
        big = (1 << 64) - 1
        return COptions(C.sizeof(COptions), self.mode, self.n_batch, self.queue_capacity, self.event_capacity,
                        int(self.slow_client_timeout * 1e9), 1 if self.prefix_cache else 0, self.min_prefix_len,
                        min(self.max_snapshot_bytes, big), min(self.swap_min_tokens, big), self.max_retained,
                        int(self.retain_ttl * 1e9))


@dataclass
class Retention:
    key: str
    release: Optional[str] = None


@dataclass
class Request:
    """crates/retrograd-infer/src/request.rs:16-47."""
    prompt: Sequence[int]
    sampling: List[E.SamplingParamsV2]
    stop: Sequence[str] = ()
    n_top_logprobs: int = 0
    logprobs: bool = False
    adapter: Optional[str] = None
    unparse_special: bool = False
    retention: Optional[Retention] = None

    @staticmethod
    def single(prompt: Sequence[int], sampling: E.SamplingParamsV2) -> "Request":
        return Request(list(prompt), [sampling])


def fake_sampling(seed: int, max_new_tokens: int) -> E.SamplingParamsV2:
    """crates/retrograd-infer/src/fake.rs:578-593: temperature 1, top-p 1, extended fields neutral."""
    return E.SamplingParamsV2(temperature=1.0, top_p=1.0, max_new_tokens=max_new_tokens, seed=seed)


@dataclass
class TopLogprob:
    token: int
    logprob: float
    piece: bytes


@dataclass
class Event:
    """crates/retrograd-infer/src/request.rs:172-257; `type` is "Token", "End" or "Error"."""
    type: str
    index: int = 0
    token: int = 0
    logprob: float = 0.0
    sampled_logprob: Optional[float] = None
    forced: bool = False
    text: str = ""
    piece: bytes = b""
    top_logprobs: List[TopLogprob] = field(default_factory=list)
    reason: Optional[str] = None
    cached_tokens: int = 0
    error: Optional[InferError] = None


class EventStream:
    """The receiving end of one request; dropping it (`close`) cancels the request at the next step."""

    def __init__(self, handle: int, owner: "Scheduler"):
        self._h, self._owner = handle, owner

    def poll(self):
        """("Ready", event) | ("Empty", None) | ("Closed", None)."""
        if not self._h:
            return "Closed", None
        ev = CEvent()
        s = _lib().retro_sched_stream_poll(self._h, C.byref(ev))
        if s == 1:
            return "Empty", None
        if s != 0:
            return "Closed", None
        if ev.type == EVENT_TOKEN:
            tops = [TopLogprob(ev.top_ids[i], ev.top_logprobs[i], C.string_at(ev.top_pieces[i], ev.top_piece_lens[i]))
                    for i in range(ev.n_top)]
            out = Event("Token", ev.index, ev.token, ev.logprob, ev.sampled_logprob if ev.has_sampled_logprob else None,
                        bool(ev.forced), C.string_at(ev.text, ev.n_text).decode("utf-8"),
                        C.string_at(ev.piece, ev.n_piece), tops)
        elif ev.type == EVENT_END:
            out = Event("End", ev.index, text=C.string_at(ev.text, ev.n_text).decode("utf-8"),
                        reason=FINISH[ev.reason], cached_tokens=ev.cached_tokens)
        else:
            out = Event("Error", error=InferError(ERROR_KINDS.get(ev.error_kind, "Failed"),
                                                  (ev.error_message or b"").decode("utf-8", "replace"),
                                                  ev.error_needed, ev.error_available))
        return "Ready", out

    def drain(self) -> List[Event]:
        """Every buffered event (does not block; pump the scheduler to produce more)."""
        out = []
        while True:
            state, ev = self.poll()
            if state != "Ready":
                return out
            out.append(ev)

    def close(self) -> None:
        if self._h:
            _lib().retro_sched_stream_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class KvStats:
    hits: int = 0
    misses: int = 0
    prefilled_cells: int = 0
    prompt_cells: int = 0
    evictions: int = 0
    swaps: int = 0
    nodes: int = 0
    resident_slots: int = 0
    snapshot_bytes: int = 0


class FakeLog:
    """Read-out of the fake backend's script and log (crates/retrograd-infer/src/fake.rs:22-75)."""

    def __init__(self, sched: "Scheduler"):
        self._s = sched

    def _ints(self, what: str, width: int):
        lib = _lib()
        n = C.c_size_t()
        _check(lib.retro_sched_fake_log(self._s._h, what.encode(), None, 0, C.byref(n)))
        buf = (C.c_int64 * max(n.value, 1))()
        _check(lib.retro_sched_fake_log(self._s._h, what.encode(), buf, n.value, C.byref(n)))
        flat = list(buf[: n.value])
        return [tuple(flat[i:i + width]) for i in range(0, len(flat), width)]

    @property
    def steps(self):
        """Every step call as rows `(slot, n_tokens, request or None)`."""
        out: List[list] = []
        for step, slot, n, request, _adapter in self._ints("steps", 5):
            while len(out) <= step:
                out.append([])
            out[step].append((slot, n, None if request < 0 else request))
        return out

    @property
    def step_adapters(self):
        out: List[list] = []
        for step, _slot, _n, _request, adapter in self._ints("steps", 5):
            while len(out) <= step:
                out.append([])
            out[step].append(adapter)
        return out

    @property
    def copies(self):
        return self._ints("copies", 4)

    @property
    def removed(self):
        return [r[0] for r in self._ints("removed", 1)]

    @property
    def request_order(self):
        return [r[0] for r in self._ints("request_order", 1)]

    def seq_pos(self, slot: int):
        """(pos_min, pos_max) of a slot of the fake pool, (-1, -1) when empty."""
        return {s: (lo, hi) for s, lo, hi in self._ints("seq_pos", 3)}[slot]

    @property
    def saves(self):
        return self._ints("saves", 3)

    @property
    def loads(self):
        return self._ints("loads", 3)

    @property
    def adapter_ops(self):
        lib = _lib()
        n = C.c_size_t()
        _check(lib.retro_sched_fake_adapter_ops(self._s._h, None, 0, C.byref(n)))
        buf = C.create_string_buffer(n.value + 1)
        _check(lib.retro_sched_fake_adapter_ops(self._s._h, buf, n.value + 1, C.byref(n)))
        out = []
        for line in buf.value.decode().splitlines():
            op, _, name = line.partition(":")
            out.append((op, name or None))
        return out

    @property
    def cells_used(self) -> int:
        v = C.c_uint64()
        _check(_lib().retro_sched_fake_cells_used(self._s._h, C.byref(v)))
        return v.value

    def set(self, key: str, value: int = 0) -> None:
        _check(_lib().retro_sched_fake_set(self._s._h, key.encode(), int(value)))

    def script(self, tokens: Sequence[int]) -> None:
        arr = (C.c_int32 * len(tokens))(*tokens)
        _check(_lib().retro_sched_fake_script(self._s._h, arr, len(tokens)))

    def bump_weights_version(self) -> None:
        self.set("bump_weights_version")

    def register_adapter(self, name: str, path: str) -> None:
        _check(_lib().retro_sched_fake_register_adapter(self._s._h, name.encode(), path.encode()))


class Scheduler:
    """The synchronous driver of the step scheduler (scheduler.rs:321-815)."""

    def __init__(self, handle: int, engine: Optional[E.Engine] = None, fake: bool = False):
        if not handle:
            raise InferError("Failed", E.last_error())
        self._h, self._engine = handle, engine
        self.fake = FakeLog(self) if fake else None

    @staticmethod
    def over_engine(engine: E.Engine, options: SchedulerOptions) -> "Scheduler":
        opts = options.to_c()
        return Scheduler(_lib().retro_scheduler_new(engine._h, C.byref(opts)), engine=engine)

    @staticmethod
    def over_trainer(trainer, options: SchedulerOptions) -> "Scheduler":
        """Scheduler::new over TrainerBackend (backend.rs:376-461): the trainer's generation context."""
        opts = options.to_c()
        return Scheduler(_lib().retro_scheduler_new_trainer(trainer._h, C.byref(opts)), engine=trainer)

    @staticmethod
    def over_fake(n_slots: int, n_ctx_seq: int, cells_total: int, vocab: int, eos: int, pieces: Sequence[str],
                  options: SchedulerOptions) -> "Scheduler":
        """FakeBackend::new (fake.rs:77-118) behind a scheduler."""
        opts = options.to_c()
        arr = (C.c_char_p * max(len(pieces), 1))(*[p.encode("utf-8") for p in pieces])
        return Scheduler(_lib().retro_scheduler_new_fake(n_slots, n_ctx_seq, cells_total, vocab, eos, arr, len(pieces),
                                                         C.byref(opts)), fake=True)

    def close(self) -> None:
        if self._h:
            _lib().retro_scheduler_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def initialize(self) -> None:
        _check(_lib().retro_scheduler_initialize(self._h))

    def submit(self, request: Request) -> EventStream:
        n = len(request.sampling)
        prompt = (C.c_int32 * max(len(request.prompt), 1))(*request.prompt)
        samp = (E.CSamplingParamsV2 * max(n, 1))()
        grammars = (C.c_char_p * max(n, 1))()
        keep = []
        for i, p in enumerate(request.sampling):
            ids = (C.c_int32 * max(len(p.logit_bias), 1))(*[b[0] for b in p.logit_bias])
            vals = (C.c_float * max(len(p.logit_bias), 1))(*[b[1] for b in p.logit_bias])
            keep += [ids, vals]
            samp[i] = E.CSamplingParamsV2(C.sizeof(E.CSamplingParamsV2), p.temperature, p.top_p, p.max_new_tokens,
                                          p.seed, p.top_k, p.min_p, p.repeat_penalty, p.frequency_penalty,
                                          p.presence_penalty, p.penalty_window, len(p.logit_bias),
                                          ids if p.logit_bias else None, vals if p.logit_bias else None, None)
            grammars[i] = p.grammar.encode() if p.grammar else None
        stops = (C.c_char_p * max(len(request.stop), 1))(*[s.encode("utf-8") for s in request.stop])
        req = CRequest(C.sizeof(CRequest), prompt if request.prompt else None, len(request.prompt),
                       samp if n else None, n, grammars, stops, len(request.stop), request.n_top_logprobs,
                       1 if request.logprobs else 0, request.adapter.encode() if request.adapter is not None else None,
                       1 if request.unparse_special else 0,
                       request.retention.key.encode() if request.retention else None,
                       request.retention.release.encode() if request.retention and request.retention.release is not None else None)
        out = C.c_void_p()
        _check(_lib().retro_scheduler_submit(self._h, C.byref(req), C.byref(out)))
        return EventStream(out.value, self)

    def pump(self) -> bool:
        progressed = C.c_uint8()
        _check(_lib().retro_scheduler_pump(self._h, C.byref(progressed)))
        return bool(progressed.value)

    def run_until_idle(self) -> None:
        _check(_lib().retro_scheduler_run_until_idle(self._h))

    def _counts(self):
        q, l = C.c_uint64(), C.c_uint64()
        _check(_lib().retro_scheduler_counts(self._h, C.byref(q), C.byref(l)))
        return q.value, l.value

    def queued_len(self) -> int:
        return self._counts()[0]

    def live_len(self) -> int:
        return self._counts()[1]

    def is_idle(self) -> bool:
        return self._counts() == (0, 0)

    def fail_queued(self) -> None:
        _check(_lib().retro_scheduler_fail_queued(self._h))

    def kv_stats(self) -> KvStats:
        st = CKvStats()
        _check(_lib().retro_scheduler_kv_stats(self._h, C.byref(st)))
        return KvStats(st.hits, st.misses, st.prefilled_cells, st.prompt_cells, st.evictions, st.swaps, st.nodes,
                       st.resident_slots, st.snapshot_bytes)

    def lend_slot(self, cells: int) -> Optional[int]:
        """scheduler.rs:746-777: a free slot with `cells` of the pool beside the dormant prefixes, or None."""
        out = C.c_int32()
        _check(_lib().retro_scheduler_lend_slot(self._h, cells, C.byref(out)))
        return None if out.value < 0 else out.value

    def queue_capacity(self) -> int:
        out = C.c_size_t()
        _check(_lib().retro_scheduler_queue_capacity(self._h, C.byref(out)))
        return out.value

    def pin_prefix(self, prefix: Sequence[int]) -> int:
        arr = (C.c_int32 * max(len(prefix), 1))(*prefix)
        pin = C.c_uint64()
        _check(_lib().retro_scheduler_pin_prefix(self._h, arr, len(prefix), C.byref(pin)))
        return pin.value

    def unpin(self, pin: int) -> bool:
        released = C.c_uint8()
        _check(_lib().retro_scheduler_unpin(self._h, pin, C.byref(released)))
        return bool(released.value)

    def load_adapter(self, name: str, path: str) -> None:
        _check(_lib().retro_scheduler_load_adapter(self._h, name.encode(), path.encode()))

    def unload_adapter(self, name: str) -> None:
        _check(_lib().retro_scheduler_unload_adapter(self._h, name.encode()))

    def set_mode(self, mode: int) -> None:
        _check(_lib().retro_scheduler_set_mode(self._h, mode))


# ---- the synchronous batch driver (crates/retrograd-infer/src/sync.rs) -----------------------------

@dataclass
class Completion:
    """sync.rs:20-37: one completion of a request, assembled from its token events."""
    tokens: List[int] = field(default_factory=list)
    logprobs: List[float] = field(default_factory=list)
    forced: List[bool] = field(default_factory=list)
    text: str = ""
    finish: Optional[str] = None


@dataclass
class RequestOutcome:
    """sync.rs:39-45: one completion per sampling entry, or the error that failed the request."""
    completions: List[Completion]
    error: Optional[InferError] = None

    def absorb(self, e: Event) -> None:
        if e.type == "Error":
            self.error = e.error
            return
        if e.index >= len(self.completions):
            self.error = InferError("Failed", "a%s event named completion %d, but the request has %d"
                                    % (" token" if e.type == "Token" else "n end", e.index, len(self.completions)))
            return
        member = self.completions[e.index]
        if e.type == "Token":
            member.tokens.append(e.token)
            member.logprobs.append(e.logprob)
            member.forced.append(e.forced)
            member.text += e.text
        else:
            member.finish = e.reason
            member.text += e.text


def run_requests(scheduler: Scheduler, requests: Sequence[Request], on_step=None) -> List[RequestOutcome]:
    """sync.rs:96-149: submits the requests in order (as the admission queue has room) and pumps until every
    one has ended, draining the streams after each step; one outcome per request in submission order. A request
    whose reservation can never fit comes back as an error in its outcome; a step failure is raised."""
    pending = list(requests)
    streams: List[EventStream] = []
    outcomes: List[RequestOutcome] = []
    capacity = scheduler.queue_capacity()
    stalled = 0
    while True:
        while pending and scheduler.queued_len() < capacity:
            request = pending.pop(0)
            streams.append(scheduler.submit(request))
            outcomes.append(RequestOutcome([Completion() for _ in request.sampling]))
        if not pending and scheduler.is_idle():
            break
        progressed = scheduler.pump()
        if on_step:
            on_step(scheduler)
        for stream, outcome in zip(streams, outcomes):
            for event in stream.drain():
                outcome.absorb(event)
        stalled = 0 if progressed else stalled + 1
        if stalled > 1024:
            raise InferError("Failed", "the scheduler made no progress with requests still queued")
    for stream, outcome in zip(streams, outcomes):
        for event in stream.drain():
            outcome.absorb(event)
    return outcomes
