"""TEST INFRASTRUCTURE - CPU oracle of the step scheduler's policy, never
imported by the product.

A pure-Python restatement of the reference's scheduling policy, written from
the Rust sources and independent of the C++ product in
retrograd_amd/csrc/sched/:

  * `PrefixTree`      crates/retrograd-infer/src/kv.rs:140-535
  * `Detokenizer`     crates/retrograd-infer/src/detok.rs:14-118
  * `FakeBackend`     crates/retrograd-infer/src/fake.rs:22-575
  * `Scheduler`       crates/retrograd-infer/src/scheduler.rs:321-1955
                      (the synchronous driver: submit / pump / run_until_idle)

Pinned by the reference's own tests, replayed in tests/test_scheduler_policy.py
(crates/retrograd-infer/src/scheduler.rs:1996-2330, src/detok.rs:120-211,
src/kv.rs tests, tests/prefix_cache.rs, tests/fake_backend.rs): every expected
value in those scenarios is the reference's, not this file's.
"""

from __future__ import annotations

import struct
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

LOCKSTEP, CONTINUOUS = 0, 1
I32_MAX = 2**31 - 1
U64_MAX = 2**64 - 1


class InferError(Exception):
    def __init__(self, kind: str, message: str = "", needed: int = 0, available: int = 0, capacity: int = 0):
        # the Display strings of error.rs:8-27 for the variants that carry no text of their own
        if kind == "KvFull" and not message:
            message = "kv pool capacity: %d cells needed, %d available" % (needed, available)
        elif kind == "QueueFull" and not message:
            message = "admission queue is full (capacity %d)" % capacity
        elif kind == "Cancelled" and not message:
            message = "request cancelled"
        super().__init__("%s: %s" % (kind, message))
        self.kind, self.message = kind, message
        self.needed, self.available, self.capacity = needed, available, capacity

    def cloned(self) -> "InferError":
        # error.rs:43-60: the backend's own error does not clone; it arrives as Failed
        kind = "Failed" if self.kind == "Backend" else self.kind
        return InferError(kind, self.message, self.needed, self.available, self.capacity)


def invalid(message: str) -> InferError:
    return InferError("InvalidArgument", message)


# --------------------------------------------------------------------------- sampling parameters

@dataclass
class Sampling:
    """retrograd-core/src/types.rs:1353-1374 with the neutral values of From<SamplingParams>."""
    temperature: float = 1.0
    top_p: float = 1.0
    max_new_tokens: int = 1
    seed: int = 0
    top_k: int = 0
    min_p: float = 0.0
    repeat_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    penalty_window: int = 0
    logit_bias: tuple = ()
    grammar_gbnf: Optional[str] = None


def _f32_total_key(x: float) -> int:
    bits = struct.unpack("<i", struct.pack("<f", x))[0]
    return bits ^ (((bits >> 31) & 0xFFFFFFFF) >> 1)


def _f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def sampling_key(s: Sampling):
    """scheduler.rs:269-293 as a sort key."""
    return (s.seed, s.max_new_tokens, _f32_total_key(s.temperature), _f32_total_key(s.top_p), s.top_k,
            _f32_total_key(s.min_p), _f32_total_key(s.repeat_penalty), _f32_total_key(s.frequency_penalty),
            _f32_total_key(s.presence_penalty), s.penalty_window,
            tuple((i, _f32_bits(b)) for i, b in s.logit_bias),
            (0, b"") if s.grammar_gbnf is None else (1, s.grammar_gbnf.encode("utf-8")))


@dataclass
class Request:
    prompt: List[int]
    sampling: List[Sampling]
    stop: List[str] = field(default_factory=list)
    n_top_logprobs: int = 0
    logprobs: bool = False
    adapter: Optional[str] = None
    unparse_special: bool = False
    retention: Optional[Tuple[str, Optional[str]]] = None     # (key, release)

    def n(self) -> int:
        return len(self.sampling)


def canonical_key(r: Request):
    """scheduler.rs:260-267"""
    return (len(r.prompt), list(r.prompt), sampling_key(r.sampling[0]))


def member_need(prompt_len: int, s: Sampling, n_ctx_seq: int) -> Optional[int]:
    if prompt_len >= n_ctx_seq:
        return None
    return prompt_len + min(s.max_new_tokens, n_ctx_seq - prompt_len)


def reservation(r: Request, n_ctx_seq: int) -> int:
    total = 0
    for s in r.sampling:
        total = min(U64_MAX, total + (member_need(len(r.prompt), s, n_ctx_seq) or 0))
    return total


def namespace(adapter: int) -> int:
    if adapter > 0:
        return adapter
    return 0 if adapter == 0 else U64_MAX


# --------------------------------------------------------------------------- streams

class Stream:
    def __init__(self, capacity: int):
        self.queue: List[dict] = []
        self.capacity = capacity
        self.senders = 0
        self.receiver_alive = True
        self.cancelled = False

    def try_send(self, event: dict) -> str:
        if not self.receiver_alive:
            return "Disconnected"
        if len(self.queue) >= self.capacity:
            return "Full"
        self.queue.append(event)
        return "Ok"

    def drop(self) -> None:          # EventStream::drop (request.rs:301-307)
        self.receiver_alive = False
        self.cancelled = True

    def drain(self) -> List[dict]:
        out, self.queue = self.queue, []
        return out

    def closed(self) -> bool:
        return not self.queue and self.senders == 0


# --------------------------------------------------------------------------- detokenizer

class Detokenizer:
    def __init__(self, stops: List[str]):
        self.stops = [s.encode("utf-8") for s in stops if s != ""]
        self.max_stop = max([len(s) for s in self.stops], default=0)
        self.pending = b""
        self.held = b""              # complete characters, UTF-8 encoded
        self.stopped = False

    def push_bytes(self, data: bytes) -> Tuple[str, bool]:
        if self.stopped:
            return "", True
        self.pending += data
        while self.pending:
            try:
                self.pending.decode("utf-8")
                self.held += self.pending
                self.pending = b""
            except UnicodeDecodeError as e:
                self.held += self.pending[:e.start]
                rest = self.pending[e.start:]
                if e.reason == "unexpected end of data":
                    self.pending = rest
                    break
                self.held += "�".encode("utf-8")
                self.pending = self.pending[e.end:]
        stop_at = None
        for stop in self.stops:
            at = self.held.find(stop)
            if at >= 0 and (stop_at is None or at < stop_at):
                stop_at = at
        if stop_at is not None:
            emitted = self.held[:stop_at]
            self.held, self.pending, self.stopped = b"", b"", True
            return emitted.decode("utf-8"), True
        hold = 0
        if self.max_stop > 1:
            for stop in self.stops:
                for k in range(len(stop) - 1, 0, -1):
                    if k > hold and len(self.held) >= k and self.held[len(self.held) - k:] == stop[:k]:
                        hold = k
                        break
        split = len(self.held) - hold
        emitted, self.held = self.held[:split], self.held[split:]
        return emitted.decode("utf-8"), False

    def finish(self) -> str:
        out = self.held + self.pending.decode("utf-8", "replace").encode("utf-8")
        self.pending, self.held = b"", b""
        return out.decode("utf-8")


# --------------------------------------------------------------------------- prefix tree

class _Node:
    __slots__ = ("edge", "parent", "depth", "slot", "snapshot", "last_use", "pins", "children")

    def __init__(self):
        self.edge: List[int] = []
        self.parent = 0
        self.depth = 0
        self.slot: Optional[int] = None
        self.snapshot: Optional[bytes] = None
        self.last_use = 0
        self.pins = 0
        self.children: Dict[int, int] = {}


def _common_len(edge: List[int], tokens: List[int]) -> int:
    n = 0
    for a, b in zip(edge, tokens):
        if a != b:
            break
        n += 1
    return n


class PrefixTree:
    def __init__(self):
        self.nodes = [_Node()]
        self.free: List[int] = []
        self.pins: Dict[int, int] = {}
        self.next_pin = 1
        self.clock = 0
        self.snapshot_bytes = 0
        self.roots: Dict[int, int] = {}

    def _root(self, ns):
        return 0 if ns == 0 else self.roots.get(ns)

    def _root_or_insert(self, ns):
        r = self._root(ns)
        if r is not None:
            return r
        r = self._alloc(_Node())
        self.nodes[r].parent = r
        self.roots[ns] = r
        return r

    def _is_root(self, node):
        return not self.nodes[node].edge

    def _tick(self):
        self.clock += 1
        return self.clock

    def _alloc(self, node):
        if self.free:
            i = self.free.pop()
            self.nodes[i] = node
            return i
        self.nodes.append(node)
        return len(self.nodes) - 1

    def _sorted_children(self, node):      # BTreeMap order
        return [self.nodes[node].children[k] for k in sorted(self.nodes[node].children)]

    def longest_prefix(self, ns, tokens, partial_ok, usable: Callable[[int, int], bool]):
        best = None
        cur = self._root(ns)
        if cur is None:
            return None
        pos = 0
        while True:
            depth = self.nodes[cur].depth
            if depth > 0 and usable(cur, depth):
                best = (cur, depth)
            nxt = None
            if pos < len(tokens) and tokens[pos] in self.nodes[cur].children:
                child = self.nodes[cur].children[tokens[pos]]
                nxt = (child, _common_len(self.nodes[child].edge, tokens[pos:]))
            if nxt is not None and nxt[1] == len(self.nodes[nxt[0]].edge):
                cur = nxt[0]
                pos += nxt[1]
                continue
            if partial_ok:
                if nxt is not None:
                    child, matched = nxt
                else:
                    kids = self._sorted_children(cur)
                    child, matched = (kids[0] if kids else None), 0
                hit = pos + matched
                if child is not None and hit > 0 and (best is None or hit > best[1]):
                    slot_node = self._deepest_slot_in_subtree(child)
                    if slot_node is not None and usable(slot_node, hit):
                        best = (slot_node, hit)
            return best

    def _deepest_slot_in_subtree(self, node):
        best = None
        stack = [node]
        while stack:
            cur = stack.pop()
            if self.nodes[cur].slot is not None and (best is None or self.nodes[cur].depth > self.nodes[best].depth):
                best = cur
            stack.extend(self._sorted_children(cur))
        return best

    def touch(self, node):
        self.nodes[node].last_use = self._tick()

    def insert(self, ns, tokens, slot):
        cur = self._root_or_insert(ns)
        pos = 0
        while pos < len(tokens):
            first = tokens[pos]
            child = self.nodes[cur].children.get(first)
            if child is not None:
                matched = _common_len(self.nodes[child].edge, tokens[pos:])
                if matched < len(self.nodes[child].edge):
                    tail = self.nodes[child].edge[matched:]
                    head = self.nodes[child].edge[:matched]
                    self.nodes[child].edge = tail
                    mid_node = _Node()
                    mid_node.edge, mid_node.parent, mid_node.depth = head, cur, self.nodes[cur].depth + matched
                    mid = self._alloc(mid_node)
                    self.nodes[mid].children[tail[0]] = child
                    self.nodes[child].parent = mid
                    self.nodes[cur].children[first] = mid
                    cur = mid
                else:
                    cur = child
                pos += matched
            else:
                leaf = _Node()
                leaf.edge, leaf.parent, leaf.depth = list(tokens[pos:]), cur, len(tokens)
                new = self._alloc(leaf)
                self.nodes[cur].children[first] = new
                cur = new
                pos = len(tokens)
        attached = (not self._is_root(cur)) and self.nodes[cur].slot is None
        if attached:
            self.nodes[cur].slot = slot
            self.nodes[cur].last_use = self._tick()
        return cur, attached

    def attach_snapshot(self, node, snapshot: bytes):
        self.snapshot_bytes += len(snapshot)
        old = self.nodes[node].snapshot
        self.nodes[node].snapshot = snapshot
        if old is not None:
            self.snapshot_bytes = max(0, self.snapshot_bytes - len(old))

    def snapshot(self, node):
        return self.nodes[node].snapshot

    def slot(self, node):
        return self.nodes[node].slot

    def detach_slot(self, node):
        self.nodes[node].slot = None

    def depth(self, node):
        return self.nodes[node].depth

    def pin_at(self, ns, tokens):
        node = self._find_exact(ns, tokens)
        return None if node is None else self.pin_node(node)

    def pin_node(self, node):
        self.nodes[node].pins += 1
        self.nodes[node].last_use = self._tick()
        pid = self.next_pin
        self.next_pin += 1
        self.pins[pid] = node
        return pid

    def unpin(self, pid):
        node = self.pins.pop(pid, None)
        if node is None:
            return False
        self.nodes[node].pins -= 1
        return True

    def _find_exact(self, ns, tokens):
        cur = self._root(ns)
        if cur is None:
            return None
        pos = 0
        while pos < len(tokens):
            child = self.nodes[cur].children.get(tokens[pos])
            if child is None:
                return None
            edge = self.nodes[child].edge
            if list(tokens[pos:pos + len(edge)]) != edge:
                return None
            cur = child
            pos += len(edge)
        return None if self._is_root(cur) else cur

    def _lru(self, eligible):
        best = None
        for i in range(1, len(self.nodes)):
            n = self.nodes[i]
            if n.pins == 0 and eligible(n) and (best is None or n.last_use < self.nodes[best].last_use):
                best = i
        return best

    def eviction_candidate(self):
        return self._lru(lambda n: n.slot is not None)

    def snapshot_eviction_candidate(self):
        return self._lru(lambda n: n.slot is None and n.snapshot is not None)

    def remove(self, node):
        snap = self.nodes[node].snapshot
        if snap is not None:
            self.snapshot_bytes = max(0, self.snapshot_bytes - len(snap))
            self.nodes[node].snapshot = None
        self.nodes[node].slot = None
        child = node
        while not self._is_root(child):
            cur = self.nodes[child]
            if cur.children or cur.slot is not None or cur.snapshot is not None or cur.pins > 0:
                break
            parent, first = cur.parent, cur.edge[0]
            del self.nodes[parent].children[first]
            self.nodes[child] = _Node()
            self.free.append(child)
            child = parent

    def resident_slots(self):
        return [n.slot for n in self.nodes if n.slot is not None]

    def resident_cells(self):
        return sum(n.depth for n in self.nodes if n.slot is not None)

    def clear(self):
        slots = self.resident_slots()
        self.nodes = [_Node()]
        self.free, self.pins, self.roots, self.snapshot_bytes = [], {}, {}, 0
        return slots

    def drop_namespace(self, ns):
        root = self._root(ns)
        if root is None:
            return []
        slots, dropped = [], []
        stack = self._sorted_children(root)
        while stack:
            node = stack.pop()
            stack.extend(self._sorted_children(node))
            if self.nodes[node].slot is not None:
                slots.append(self.nodes[node].slot)
            if self.nodes[node].snapshot is not None:
                self.snapshot_bytes = max(0, self.snapshot_bytes - len(self.nodes[node].snapshot))
            dropped.append(node)
        for node in dropped:
            self.nodes[node].pins = 0
        self.pins = {k: v for k, v in self.pins.items() if self.nodes[v].pins != 0}
        for node in dropped:
            self.nodes[node] = _Node()
            self.free.append(node)
        self.nodes[root].children.clear()
        if root != 0:
            del self.roots[ns]
            self.nodes[root] = _Node()
            self.free.append(root)
        return slots

    def node_count(self):
        return len(self.nodes) - 1 - len(self.roots) - len(self.free)

    def resident_slot_count(self):
        return len(self.resident_slots())


# --------------------------------------------------------------------------- fake backend

PARTIAL_ONLY = 1


class FakeBackend:
    def __init__(self, n_slots, n_ctx_seq, cells_total, vocab, eos, pieces):
        self.n_slots, self.n_ctx_seq, self.cells_total, self.vocab, self.eos = n_slots, n_ctx_seq, cells_total, vocab, eos
        self.pieces = list(pieces)
        self.eog_after: Optional[int] = None
        self.script: Optional[List[int]] = None
        self.slots: List[Optional[Tuple[int, int]]] = [None] * n_slots
        self.requests: Dict[int, int] = {}
        self.steps: List[list] = []
        self.step_adapters: List[list] = []
        self.copies: List[tuple] = []
        self.removed: List[int] = []
        self.request_order: List[int] = []
        self.saves: List[tuple] = []
        self.loads: List[tuple] = []
        self.kv_unified_flag = True
        self.recurrent = False
        self.weights_version_value = 0
        self.fingerprint = 0xFACE
        self.adapters: Dict[str, str] = {}
        self.active: Optional[str] = None
        self.adapter_ops: List[tuple] = []
        self.row_adapters_enabled = False
        self.row_adapters: Dict[int, str] = {}
        self.next_row_adapter = 1
        self.fail_after_steps = -1

    def bump_weights_version(self):
        self.weights_version_value += 1

    def register_adapter(self, name, path):
        self.adapters[name] = path
        self.adapter_ops.append(("load", name))

    def apply_adapter(self, name):
        if name is None:
            self.active = None
        elif name in self.adapters:
            self.active = name
        else:
            raise invalid("no adapter registered under '%s'" % name)
        self.adapter_ops.append(("activate", self.active))
        self.slots = [None] * self.n_slots
        self.bump_weights_version()

    def _encode_snapshot(self, slot, flags):
        span = self.slots[slot] if 0 <= slot < self.n_slots else None
        if span is None:
            return None
        return struct.pack("<IIii", 0x5EED, flags, span[0], span[1])

    def cells_used(self):
        return sum(hi - lo + 1 for lo, hi in (s for s in self.slots if s is not None))

    def _sample_token(self, request, generated):
        if self.eog_after == generated:
            return self.eos
        if self.script:
            return self.script[generated % len(self.script)]
        vocab = max(max(self.vocab - 1, 0), 1)
        return (request * 31 + generated * 7 + 1) % vocab        # rem_euclid

    def step(self, rows):
        if not rows:
            raise invalid("a step requires at least one row")
        if sum(len(r["tokens"]) for r in rows) == 0:
            raise invalid("a step row requires tokens")
        self.steps.append([(r["slot"], len(r["tokens"]), r["request"] if r["sample"] else None) for r in rows])
        self.step_adapters.append([r["adapter"] for r in rows])
        for r in rows:
            if r["adapter"] > 0 and r["adapter"] not in self.row_adapters:
                raise invalid("step row adapter %d is not a loaded per-row adapter" % r["adapter"])
        used = self.cells_used()
        for r in rows:
            slot, n = r["slot"], len(r["tokens"])
            if slot < 0 or slot >= self.n_slots:
                raise invalid("step row slot out of range")
            if n == 0:
                raise invalid("a step row requires at least one token")
            end = r["pos0"] + n
            if end > I32_MAX:
                raise InferError("Overflow", "position range overflows i32")
            if end > self.n_ctx_seq:
                raise invalid("a step row decodes past the per-sequence context")
            span = self.slots[slot]
            if span is None:
                used += n
            elif r["pos0"] == span[1] + 1:
                used += n
            elif r["pos0"] >= span[0] and end - 1 <= span[1]:
                pass
            else:
                raise invalid("a step row leaves a gap in its slot's resident span")
            if r["sample"] and r["request"] < 0:
                raise invalid("a sampling step row requires a request id >= 0")
        if used > self.cells_total:
            raise InferError("Backend", "the fake KV pool is full")
        out = []
        for r in rows:
            end = r["pos0"] + len(r["tokens"])
            span = self.slots[r["slot"]]
            self.slots[r["slot"]] = (r["pos0"], end - 1) if span is None else (min(span[0], r["pos0"]), max(span[1], end - 1))
            if not r["sample"]:
                out.append(dict(sampled=False, token=0, logprob=0.0, forced=False, sampled_logprob=0.0, top=[]))
                continue
            generated = self.requests.get(r["request"], 0)
            if r["request"] not in self.request_order:
                self.request_order.append(r["request"])
            token = self._sample_token(r["request"], generated)
            self.requests[r["request"]] = generated + 1
            n_top = min(r["n_top_logprobs"], self.vocab)
            out.append(dict(sampled=True, token=token, logprob=-0.5, forced=False,
                            sampled_logprob=-0.7 if r["want_logprob"] else 0.0,
                            top=[(k, -1.0 - k) for k in range(n_top)]))
        if self.fail_after_steps == 0:
            self.fail_after_steps = -1
            raise InferError("Backend", "partial decode failure")
        if self.fail_after_steps > 0:
            self.fail_after_steps -= 1
        return out

    def seq_rm(self, slot, p0, p1):
        if slot < 0 or slot >= self.n_slots:
            raise invalid("seq_rm slot out of range")
        self.removed.append(slot)
        if p0 == -1 and p1 == -1:
            self.slots[slot] = None
        elif self.slots[slot] is not None:
            lo, hi = self.slots[slot]
            lo = p1 if p0 <= lo else lo
            hi = lo - 1 if (p1 >= hi or p1 < 0) else hi
            self.slots[slot] = None if lo > hi else (lo, hi)

    def seq_cp(self, src, dst, p0, p1):
        if not (0 <= src < self.n_slots and 0 <= dst < self.n_slots):
            raise invalid("seq_cp slot out of range")
        partial = not (p0 == -1 and p1 == -1)
        if partial and not self.kv_unified_flag:
            raise invalid("seq_cp: a partial range between streams of a partitioned pool is unsupported")
        self.copies.append((src, dst, p0, p1))
        span = self.slots[src]
        if span is None:
            raise invalid("seq_cp source slot is empty")
        if self.slots[dst] is not None:
            raise invalid("seq_cp destination slot is not empty")
        if not partial:
            self.slots[dst] = span
        else:
            lo = max(span[0], 0 if p0 < 0 else p0)
            hi = span[1] if p1 < 0 else min(span[1], p1 - 1)
            self.slots[dst] = (lo, hi) if lo <= hi else None

    def seq_pos(self, slot):
        if slot < 0 or slot >= self.n_slots:
            raise invalid("seq_pos slot out of range")
        return self.slots[slot] if self.slots[slot] is not None else (-1, -1)

    def seq_save_len(self, slot, flags):
        if slot < 0 or slot >= self.n_slots:
            raise invalid("seq_save slot out of range")
        if flags == PARTIAL_ONLY and self.recurrent:
            return 8
        if flags not in (0, PARTIAL_ONLY):
            raise invalid("unknown snapshot flags")
        enc = self._encode_snapshot(slot, flags)
        return len(enc) if enc is not None else 0

    def seq_save(self, slot, flags, capacity):
        if flags == PARTIAL_ONLY and self.recurrent:
            enc = struct.pack("<II", 0x5EED, PARTIAL_ONLY)
        else:
            enc = self._encode_snapshot(slot, flags)
            if enc is None:
                raise invalid("seq_save slot is empty")
        if capacity < len(enc):
            raise invalid("save buffer too small")
        self.saves.append((slot, flags, len(enc)))
        return enc

    def seq_load(self, slot, flags, data):
        if slot < 0 or slot >= self.n_slots:
            raise invalid("seq_load slot out of range")
        self.loads.append((slot, flags, len(data)))
        if flags == PARTIAL_ONLY and self.recurrent:
            return len(data)
        if len(data) < 16 or struct.unpack("<I", data[:4])[0] != 0x5EED:
            raise invalid("corrupted snapshot")
        lo, hi = struct.unpack("<ii", data[8:16])
        self.slots[slot] = (lo, hi)
        return len(data)

    def kv_unified(self):
        return self.kv_unified_flag

    def is_hybrid(self):
        return self.recurrent

    def cache_key(self):
        return (self.fingerprint, self.weights_version_value, int(self.kv_unified_flag))

    def memory(self):
        used = self.cells_used()
        return dict(n_slots=self.n_slots, cells_total=self.cells_total, cells_used=used)

    def request_free(self, request):
        self.requests.pop(request, None)

    def is_eog_token(self, token):
        return token == self.eos

    def detokenize_bytes(self, tokens, unparse_special):
        out = b""
        for t in tokens:
            if t == self.eos and not unparse_special:
                continue
            out += (self.pieces[t] if 0 <= t < len(self.pieces) else "<%d>" % t).encode("utf-8")
        return out

    def context_size(self):
        return self.n_ctx_seq

    def vocab_size(self):
        return self.vocab

    def load_adapter(self, name, path):
        if name == "":
            raise invalid("adapter name must not be empty")
        self.register_adapter(name, path)

    def activate_adapter(self, name):
        self.apply_adapter(name)

    def active_adapter(self):
        return self.active

    def supports_row_adapters(self):
        return self.row_adapters_enabled

    def load_row_adapter(self, path, scale):
        if not self.row_adapters_enabled:
            raise InferError("Failed", "per-row adapters are disabled")
        aid = self.next_row_adapter
        self.next_row_adapter += 1
        self.row_adapters[aid] = path
        self.adapter_ops.append(("load_row", str(aid)))
        return aid

    def unload_row_adapter(self, aid):
        if aid not in self.row_adapters:
            raise invalid("no per-row adapter %d" % aid)
        del self.row_adapters[aid]
        self.adapter_ops.append(("unload_row", str(aid)))


# --------------------------------------------------------------------------- scheduler

@dataclass
class Options:
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


class _Member:
    pass


class _Group:
    pass


class Scheduler:
    def __init__(self, backend: FakeBackend, options: Options):
        self.backend = backend
        self.o = options
        self.o.queue_capacity = max(self.o.queue_capacity, 1)
        self.queue: List[Tuple[Request, Stream]] = []
        self.live: List[_Group] = []
        self.n_slots = 0
        self.next_request_id = 1
        self.out: List[dict] = []
        self.decode_cursor = 0
        self.prefill_turn = False
        self.kv = PrefixTree()
        self.kv_key = None
        self.stats = dict(hits=0, misses=0, prefilled_cells=0, prompt_cells=0, evictions=0, swaps=0)
        self.retained: Dict[str, Tuple[int, float, int]] = {}
        self._retained_seq = 0
        self.active_adapter: Optional[str] = None
        self.row_adapters: Dict[str, int] = {}
        self.retiring: List[int] = []
        self.unloaded_adapters = set()

    # -- helpers
    def _send_bounded(self, stream: Stream, event: dict) -> bool:
        started = time.monotonic()
        while True:
            r = stream.try_send(event)
            if r == "Ok":
                return True
            if r == "Disconnected":
                return False
            if time.monotonic() - started >= self.o.slow_client_timeout:
                return False
            time.sleep(0.001)

    def kv_stats(self) -> dict:
        out = dict(self.stats)
        out.update(nodes=self.kv.node_count(), resident_slots=self.kv.resident_slot_count(),
                   snapshot_bytes=self.kv.snapshot_bytes)
        return out

    def live_len(self) -> int:
        return sum(1 for g in self.live for m in g.members if m.live)

    def queued_len(self) -> int:
        return len(self.queue)

    def is_idle(self) -> bool:
        return not self.queue and not self.live

    # -- adapters (scheduler.rs:454-532)
    def load_adapter(self, name, path):
        if name == "":
            raise invalid("an adapter name must not be empty")
        if self.backend.supports_row_adapters():
            try:
                aid = self.backend.load_row_adapter(path, 1.0)
            except InferError:
                aid = None
            if aid is not None:
                self.unloaded_adapters.discard(name)
                old = self.row_adapters.get(name)
                self.row_adapters[name] = aid
                if old is not None:
                    self.retiring.append(old)
                    self._release_retired()
                return
        self.backend.load_adapter(name, path)
        self.unloaded_adapters.discard(name)
        old = self.row_adapters.pop(name, None)
        if old is not None:
            self.retiring.append(old)
            self._release_retired()

    def unload_adapter(self, name):
        if name not in self.row_adapters:
            raise invalid("no per-row adapter is loaded under '%s'" % name)
        aid = self.row_adapters.pop(name)
        self.unloaded_adapters.add(name)
        self.retiring.append(aid)
        self._release_retired()

    def _release_retired(self):
        index = 0
        while index < len(self.retiring):
            aid = self.retiring[index]
            if any(g.adapter == aid for g in self.live):
                index += 1
                continue
            for slot in self.kv.drop_namespace(namespace(aid)):
                self.backend.seq_rm(slot, -1, -1)
            self.backend.unload_row_adapter(aid)
            self.retiring[index] = self.retiring[-1]      # swap_remove
            self.retiring.pop()

    def _row_adapter(self, r: Request) -> int:
        if r.adapter is not None and r.adapter in self.row_adapters:
            return self.row_adapters[r.adapter]
        return 0

    def _serial_adapter(self, r: Request) -> Optional[str]:
        if r.adapter is not None and r.adapter not in self.row_adapters:
            return r.adapter
        return None

    def _ensure_adapter(self, wanted):
        if self.backend.active_adapter() != wanted:
            self.backend.activate_adapter(wanted)
            self.active_adapter = wanted
            self._refresh_key()

    # -- pins and retentions (scheduler.rs:534-612)
    def pin_prefix(self, prefix):
        self._refresh_key()
        pin = self.kv.pin_at(0, list(prefix))
        if pin is None:
            raise invalid("no resident prefix node at exactly that token path")
        return pin

    def unpin(self, pin):
        return self.kv.unpin(pin)

    def _refresh_key(self):
        key = self.backend.cache_key()
        if self.kv_key != key:
            for slot in self.kv.clear():
                self.backend.seq_rm(slot, -1, -1)
            self.retained.clear()
            self.kv_key = key

    def _retain(self, key, node):
        old = self.retained.pop(key, None)
        if old is not None:
            self.kv.unpin(old[0])
        cap = min(self.o.max_retained, self.n_slots // 4)
        if cap == 0:
            return
        while len(self.retained) >= cap and self._release_oldest_retained():
            pass
        pin = self.kv.pin_node(node)
        self.retained[key] = (pin, time.monotonic(), self._retained_seq)
        self._retained_seq += 1

    def _release_retained(self, key):
        r = self.retained.pop(key, None)
        return False if r is None else self.kv.unpin(r[0])

    def _release_oldest_retained(self):
        if not self.retained:
            return False
        key = min(self.retained, key=lambda k: (self.retained[k][1], self.retained[k][2]))
        return self._release_retained(key)

    def _release_expired_retained(self):
        now = time.monotonic()
        for key in list(self.retained):
            pin, since, _ = self.retained[key]
            if not (now - since < self.o.retain_ttl):
                self.kv.unpin(pin)
                del self.retained[key]

    # -- driver (scheduler.rs:665-815)
    def initialize(self):
        mem = self.backend.memory()
        self.n_slots = mem["n_slots"]
        for slot in range(self.n_slots):
            self.backend.seq_rm(slot, -1, -1)
        self.active_adapter = self.backend.active_adapter()

    def submit(self, request: Request) -> Stream:
        validate(request)
        if len(self.queue) >= self.o.queue_capacity:
            raise InferError("QueueFull", capacity=self.o.queue_capacity)
        stream = Stream(max(self.o.event_capacity, request.n() + 2))
        stream.senders += 1
        self.queue.append((request, stream))
        return stream

    def pump(self) -> bool:
        before = (len(self.queue), self.live_len())
        try:
            stepped = self._step_once()
            return stepped or (len(self.queue), self.live_len()) != before
        except InferError as error:
            self._fail_all(error)
            raise

    def run_until_idle(self):
        stalled = 0
        while not self.is_idle():
            if self.pump():
                stalled = 0
            else:
                stalled += 1
                if stalled > 1024:
                    raise InferError("Failed", "the scheduler made no progress with requests still queued")

    def lend_slot(self, cells: int) -> Optional[int]:
        """scheduler.rs:746-777."""
        if self.live:
            raise InferError("Failed", "a slot can only be lent while no sequence is live")
        while True:
            slots_left, cells_left = self._capacity()
            if slots_left > 0 and cells_left >= cells:
                held = set(self.kv.resident_slots())
                for slot in range(self.n_slots):
                    if slot not in held:
                        return slot
                return None
            if not self._evict_one_lru():
                return None

    def queue_capacity(self) -> int:
        return self.o.queue_capacity

    def fail_queued(self):
        while self.queue:
            _, stream = self.queue.pop(0)
            stream.try_send(dict(type="Error", error=InferError("Cancelled")))
            stream.senders -= 1

    def _drop_dead_groups(self):
        self.live = [g for g in self.live if any(m.live for m in g.members)]

    def _step_once(self) -> bool:
        kept = []
        for r, stream in self.queue:
            if stream.cancelled:
                stream.senders -= 1
            else:
                kept.append((r, stream))
        self.queue = kept
        self._remove_cancelled()
        if self.retiring:
            self._release_retired()
        self._admit()
        self._advance_phases()
        if not self.live:
            return False
        rows, kinds, total_tokens = self._compose()
        if not rows:
            return False
        try:
            self.out = self.backend.step(rows)
        except InferError as error:
            error = self._classify_step_error(error, total_tokens)
            self._rollback(kinds)
            raise error
        for index, kind in enumerate(kinds):
            if kind[0] == "Decode":
                self._emit_sampled(kind[1], kind[2], self.out[index])
            elif kind[0] == "Terminal":
                self._emit_sampled(kind[1], kind[2], self.out[index])
                g = self.live[kind[1]]
                if g.phase == "Terminal":
                    g.pos = max(g.pos, kind[2] + 1)
                    if g.pos >= len(g.members):
                        g.phase = "Decode"
            else:
                _, group, end, sampled_member = kind
                g = self.live[group]
                if g.phase == "Prefill":
                    g.pos = end
                if sampled_member is not None:
                    self._emit_sampled(group, sampled_member, self.out[index])
        self._drop_dead_groups()
        if self.retiring:
            self._release_retired()
        return True

    # -- compose (scheduler.rs:933-1089)
    def _compose(self):
        n_batch = max(self.o.n_batch, 1)
        used = 0
        rows, kinds = [], []
        prefill_active = any(g.phase != "Decode" for g in self.live)
        allow_decode = self.o.mode == CONTINUOUS or not prefill_active
        decode_list = []
        if allow_decode:
            for gi, g in enumerate(self.live):
                if g.phase != "Decode":
                    continue
                for mi, m in enumerate(g.members):
                    if m.live:
                        decode_list.append((gi, mi))
        if self.o.mode == CONTINUOUS and prefill_active:
            if n_batch == 1:
                self.prefill_turn = not self.prefill_turn
                decode_budget = 0 if self.prefill_turn else 1
            else:
                decode_budget = n_batch - 1
        else:
            decode_budget = n_batch
        if decode_list:
            start = self.decode_cursor % len(decode_list)
            decode_list = decode_list[start:] + decode_list[:start]
            count = min(decode_budget, len(decode_list))
            self.decode_cursor = (start + count) % len(decode_list)
            decode_list = decode_list[:count]
        used += len(decode_list)

        def position(pos):
            if pos > I32_MAX:
                raise InferError("Overflow", "a step position does not fit i32")
            return pos

        for gi, mi in decode_list:
            g = self.live[gi]
            m = g.members[mi]
            rows.append(dict(request=m.request_id, slot=m.slot, tokens=[m.next_token],
                             pos0=position(len(g.prompt) + m.generated - 1), sample=True, sampling=m.sampling,
                             n_top_logprobs=m.n_top_logprobs, want_logprob=m.want_logprob, adapter=g.adapter))
            kinds.append(("Decode", gi, mi))
        for gi, g in enumerate(self.live):
            if used >= n_batch:
                break
            if g.phase == "Prefill":
                remaining = n_batch - used
                chunk = min(remaining, g.prefix_end - g.pos)
                if chunk == 0:
                    continue
                end = g.pos + chunk
                single = len(g.members) == 1
                sampled_member = 0 if (single and end == len(g.prompt)) else None
                leader = g.members[g.leader]
                sampled = sampled_member is not None
                rows.append(dict(request=leader.request_id, slot=leader.slot, tokens=g.prompt[g.pos:end],
                                 pos0=position(g.pos), sample=sampled, sampling=leader.sampling,
                                 n_top_logprobs=leader.n_top_logprobs if sampled else 0,
                                 want_logprob=sampled and leader.want_logprob, adapter=g.adapter))
                kinds.append(("Prefill", gi, end, sampled_member))
                used += chunk
            elif g.phase == "Terminal":
                last = len(g.prompt) - 1
                mi = g.pos
                while mi < len(g.members) and used < n_batch:
                    m = g.members[mi]
                    if not m.live:
                        mi += 1
                        continue
                    rows.append(dict(request=m.request_id, slot=m.slot, tokens=g.prompt[last:], pos0=position(last),
                                     sample=True, sampling=m.sampling, n_top_logprobs=m.n_top_logprobs,
                                     want_logprob=m.want_logprob, adapter=g.adapter))
                    kinds.append(("Terminal", gi, mi))
                    used += 1
                    mi += 1
        return rows, kinds, used

    def _advance_phases(self):
        for g in self.live:
            done = g.phase == "Prefill" and g.pos == g.prefix_end
            if done:
                if len(g.members) > 1:
                    leader_slot = g.members[g.leader].slot
                    slots = [m.slot for m in g.members if m.live and m.slot != leader_slot]
                    if g.prefix_end > 0:
                        for slot in slots:
                            self.backend.seq_cp(leader_slot, slot, -1, -1)
                    g.phase, g.pos = "Terminal", 0
                else:
                    g.phase = "Decode"
            elif g.phase == "Terminal" and all(not m.live for m in g.members[g.pos:]):
                g.phase = "Decode"

    # -- admission (scheduler.rs:1124-1404)
    def _admit(self):
        if not self.queue:
            return
        self._refresh_key()
        self._release_expired_retained()
        while self.kv.snapshot_bytes > self.o.max_snapshot_bytes:
            node = self.kv.snapshot_eviction_candidate()
            if node is None:
                break
            self.kv.remove(node)
            self.stats["evictions"] += 1
        n_ctx_seq = self.backend.context_size()
        vocab = self.backend.vocab_size()
        mem = self.backend.memory()
        self.n_slots = mem["n_slots"]
        cells_total = mem["cells_total"]
        index = 0
        while index < len(self.queue):
            r, stream = self.queue[index]
            prompt_too_long = len(r.prompt) >= n_ctx_seq
            too_many_members = r.n() > self.n_slots
            top_too_wide = r.n_top_logprobs > vocab
            invalid_token = any(t < 0 or t >= vocab for t in r.prompt)
            invalid_bias = any(t < 0 or t >= vocab for s in r.sampling for t, _ in s.logit_bias)
            need = reservation(r, n_ctx_seq)
            if prompt_too_long or too_many_members or top_too_wide or invalid_token or invalid_bias or need > cells_total:
                self.queue.pop(index)
                if prompt_too_long:
                    message = ("the prompt (%d tokens) leaves no room to generate in the per-sequence context (%d)"
                               % (len(r.prompt), n_ctx_seq))
                elif too_many_members:
                    message = "the request asks for %d completions but the pool has %d slots" % (r.n(), self.n_slots)
                elif top_too_wide:
                    message = "n_top_logprobs exceeds the vocabulary (%d)" % vocab
                elif invalid_bias:
                    message = "logit_bias token ids must be in 0..%d" % vocab
                elif invalid_token:
                    message = "prompt tokens must be in 0..%d" % vocab
                else:
                    message = ("the reservation (prompt + max_new_tokens = %d cells) exceeds the KV pool of %d cells"
                               % (need, cells_total))
                stream.try_send(dict(type="Error", error=invalid(message)))
                stream.senders -= 1
                continue
            index += 1
        if not self.queue:
            return
        kept = []
        for r, stream in self.queue:
            if r.adapter is not None and r.adapter in self.unloaded_adapters:
                stream.try_send(dict(type="Error", error=invalid("no adapter is loaded under '%s'" % r.adapter)))
                stream.senders -= 1
            else:
                kept.append((r, stream))
        self.queue = kept
        if not self.queue:
            return
        target = self._serial_adapter(self.queue[0][0]) if not self.live else self.active_adapter
        candidates = [q for q in self.queue if self._serial_adapter(q[0]) == target]
        rest = [q for q in self.queue if self._serial_adapter(q[0]) != target]
        if not self.live:
            try:
                self._ensure_adapter(target)
            except InferError as error:
                for _, stream in candidates:
                    stream.try_send(dict(type="Error", error=error.cloned()))
                    stream.senders -= 1
                self.queue = rest
                return
        self.queue = candidates
        try:
            self._admit_candidates(n_ctx_seq)
        finally:
            leftover = self.queue
            self.queue = rest + leftover

    def _admit_candidates(self, n_ctx_seq):
        evictions_left = [self.n_slots + 1]
        if self.o.mode == LOCKSTEP:
            if self.live:
                return
            pending, wave_pins = [], []
            held_slots, held_cells = 0, 0
            while True:
                fit = self._front_fits(n_ctx_seq, held_slots, held_cells, evictions_left)
                if fit is None:
                    break
                members, need, node = fit
                held_slots += members
                held_cells += need
                if node is not None:
                    wave_pins.append(self.kv.pin_node(node))
                pending.append(self.queue.pop(0))
            pending.sort(key=lambda q: canonical_key(q[0]))
            failure = None
            while pending and failure is None:
                run_end = 1
                while (run_end < len(pending) and pending[run_end][0].prompt == pending[0][0].prompt
                       and pending[run_end][0].adapter == pending[0][0].adapter):
                    run_end += 1
                run, pending = pending[:run_end], pending[run_end:]
                try:
                    self._admit_group(run, n_ctx_seq)
                except InferError as error:
                    failure = error
            for pin in wave_pins:
                self.kv.unpin(pin)
            if failure is not None:
                raise failure
        else:
            while self._front_fits(n_ctx_seq, 0, 0, evictions_left) is not None:
                self._admit_group([self.queue.pop(0)], n_ctx_seq)

    def _capacity(self):
        mem = self.backend.memory()
        used_slots = self.live_len() + self.kv.resident_slot_count()
        reserved = sum(g.reserved for g in self.live)
        committed = max(mem["cells_used"], min(U64_MAX, reserved + self.kv.resident_cells()))
        return max(self.n_slots - used_slots, 0), max(mem["cells_total"] - committed, 0)

    def _front_fits(self, n_ctx_seq, held_slots, held_cells, evictions_left):
        while True:
            if not self.queue:
                return None
            r = self.queue[0][0]
            members = r.n()
            ns = namespace(self._row_adapter(r))
            hit = self._hit_candidate(ns, r.prompt)
            shared = hit[1] * members if hit is not None else 0
            need = max(reservation(r, n_ctx_seq) - shared, 0)
            slots_left, cells_left = self._capacity()
            if held_slots + members <= slots_left and held_cells + need <= cells_left:
                return members, need, (hit[0] if hit is not None else None)
            if evictions_left[0] == 0:
                return None
            if not self._evict_one_lru():
                if not self._release_oldest_retained():
                    return None
                continue
            evictions_left[0] -= 1

    def _evict_one_lru(self):
        node = self.kv.eviction_candidate()
        if node is None:
            return False
        slot = self.kv.slot(node)
        if self.kv.depth(node) >= self.o.swap_min_tokens:
            try:
                save_len = self.backend.seq_save_len(slot, 0)
            except InferError:
                save_len = 0
            if save_len > 0 and self.kv.snapshot_bytes + save_len <= self.o.max_snapshot_bytes:
                try:
                    data = self.backend.seq_save(slot, 0, save_len)
                    self.kv.attach_snapshot(node, data)
                    self.stats["swaps"] += 1
                except InferError:
                    pass
        self.backend.seq_rm(slot, -1, -1)
        self.kv.detach_slot(node)
        if self.kv.snapshot(node) is None:
            self.kv.remove(node)
        self.stats["evictions"] += 1
        return True

    # -- prefix hits (scheduler.rs:1446-1522)
    def _hit_candidate(self, ns, prompt):
        if not self.o.prefix_cache or len(prompt) < 2:
            return None
        partial_ok = self.backend.kv_unified() and not self.backend.is_hybrid()
        last = len(prompt) - 1

        def usable(node, hit):
            applied = min(hit, last)
            depth = self.kv.depth(node)
            if applied == 0 or (applied < depth and not partial_ok):
                return False
            slot = self.kv.slot(node)
            if slot is not None:
                try:
                    return self.backend.seq_pos(slot) == (0, depth - 1)
                except InferError:
                    return False
            return self.kv.snapshot(node) is not None and applied == depth

        found = self.kv.longest_prefix(ns, list(prompt), partial_ok, usable)
        return None if found is None else (found[0], min(found[1], last))

    def _apply_cache_hit(self, ns, prompt, leader_slot):
        found = self._hit_candidate(ns, prompt)
        if found is None:
            return 0
        node, hit = found
        src = self.kv.slot(node)
        if src is not None and hit == self.kv.depth(node):
            self.backend.seq_cp(src, leader_slot, -1, -1)
        elif src is not None:
            self.backend.seq_cp(src, leader_slot, 0, hit)
        else:
            self.backend.seq_load(leader_slot, 0, self.kv.snapshot(node))
        self.kv.touch(node)
        return hit

    # -- placing a group (scheduler.rs:1526-1650)
    def _admit_group(self, group, n_ctx_seq):
        prompt = list(group[0][0].prompt)
        adapter = self._row_adapter(group[0][0])
        n_members = sum(r.n() for r, _ in group)
        prefix_end = len(prompt) - 1 if n_members > 1 else len(prompt)
        members = []
        used = [False] * self.n_slots
        for g in self.live:
            for m in g.members:
                if m.live and m.slot < self.n_slots:
                    used[m.slot] = True
        for slot in self.kv.resident_slots():
            if slot < self.n_slots:
                used[slot] = True
        try:
            for request, stream in group:
                retention = request.retention
                for index, sampling in enumerate(request.sampling):
                    slot = used.index(False)
                    used[slot] = True
                    request_id = self.next_request_id

                    def bump():
                        self.next_request_id = 1 if self.next_request_id == I32_MAX else self.next_request_id + 1

                    bump()
                    while (any(m.live and m.request_id == self.next_request_id
                               for m in [m for g in self.live for m in g.members] + members)
                           or self.next_request_id == request_id):
                        bump()
                    m = _Member()
                    m.slot, m.request_id, m.index, m.sampling = slot, request_id, index, sampling
                    m.want_logprob = request.logprobs or request.n_top_logprobs > 0
                    m.limit = min(sampling.max_new_tokens, n_ctx_seq - len(prompt))
                    m.reserved_share = 0
                    m.generated, m.next_token, m.history, m.live = 0, 0, [], True
                    m.n_top_logprobs = request.n_top_logprobs
                    m.unparse_special = request.unparse_special
                    m.detok = Detokenizer(list(request.stop))
                    m.events = stream
                    stream.senders += 1
                    m.retention, retention = retention, None
                    members.append(m)
                stream.senders -= 1          # the queued envelope's own sending end
            if self.o.mode == LOCKSTEP:
                slots = sorted(m.slot for m in members)
                members.sort(key=lambda m: sampling_key(m.sampling))
                for m, slot in zip(members, slots):
                    m.slot = slot
            leader_slot = members[0].slot
            cache_hit = self._apply_cache_hit(namespace(adapter), prompt, leader_slot)
        except InferError:
            for m in members:                 # the half-built group is dropped with its senders
                m.events.senders -= 1
            raise
        prefill_from = min(cache_hit, prefix_end)
        for m in members:
            m.reserved_share = (len(prompt) - cache_hit) + m.limit
        g = _Group()
        g.prompt, g.adapter, g.prefix_end, g.leader = prompt, adapter, prefix_end, 0
        g.reserved = sum(m.reserved_share for m in members)
        g.cache_hit, g.members = cache_hit, members
        g.phase, g.pos = "Prefill", prefill_from
        if cache_hit > 0:
            self.stats["hits"] += 1
        else:
            self.stats["misses"] += 1
        self.stats["prompt_cells"] += len(prompt)
        self.stats["prefilled_cells"] += prefix_end - prefill_from
        self.live.append(g)

    # -- emit and finish (scheduler.rs:1654-1854)
    def _emit_sampled(self, group, member, produced):
        g = self.live[group]
        m = g.members[member]
        if m.events.cancelled:
            return self._finish_member(group, member, "Cancelled")
        if not produced["sampled"]:
            raise InferError("Failed", "a sampling step row produced no token")
        m.generated += 1
        m.next_token = produced["token"]
        m.history.append(produced["token"])
        if m.unparse_special and self.backend.is_eog_token(produced["token"]):
            piece = b""
        else:
            piece = self.backend.detokenize_bytes([produced["token"]], m.unparse_special)
        text, stop_hit = m.detok.push_bytes(piece)
        tops = []
        if m.n_top_logprobs > 0:
            for token, logprob in produced["top"]:
                try:
                    tp = self.backend.detokenize_bytes([token], m.unparse_special)
                except InferError:
                    tp = b""
                tops.append((token, logprob, tp))
        event = dict(type="Token", index=m.index, token=produced["token"], logprob=produced["logprob"],
                     sampled_logprob=produced["sampled_logprob"] if m.want_logprob else None,
                     forced=produced["forced"], text=text, piece=piece, top_logprobs=tops)
        send_failed = not self._send_bounded(m.events, event)
        if send_failed:
            reason = "Cancelled"
        elif stop_hit:
            reason = "Stop"
        elif self.backend.is_eog_token(produced["token"]):
            reason = "Eog"
        elif m.generated >= m.limit:
            reason = "MaxTokens" if m.limit >= m.sampling.max_new_tokens else "ContextFull"
        else:
            reason = None
        if reason is not None:
            self._finish_member(group, member, reason)

    def _finish_member(self, group, member, reason):
        g = self.live[group]
        ns = namespace(g.adapter)
        m = g.members[member]
        if not m.live:
            return
        g.reserved = max(g.reserved - m.reserved_share, 0)
        m.live = False
        text = m.detok.finish()
        path = g.prompt + m.history
        events, m.events_taken = m.events, True
        retention, m.retention = m.retention, None
        if reason == "Cancelled":
            events.cancelled = True
        if reason != "Cancelled":
            ok = self._send_bounded(events, dict(type="End", index=m.index, reason=reason, text=text,
                                                 cached_tokens=g.cache_hit))
            if not ok:
                events.cancelled = True
        try:
            pos_min, pos_max = self.backend.seq_pos(m.slot)
            resident = pos_max + 1 if pos_min == 0 else 0
            node = None
            if self.o.prefix_cache and resident > 0 and resident >= self.o.min_prefix_len and resident <= len(path):
                node, attached = self.kv.insert(ns, path[:resident], m.slot)
                if not attached:
                    self.backend.seq_rm(m.slot, -1, -1)
            else:
                self.backend.seq_rm(m.slot, -1, -1)
            self.backend.request_free(m.request_id)
            if retention is not None and reason != "Cancelled":
                key, release = retention
                if release is not None:
                    self._release_retained(release)
                if node is not None:
                    self._retain(key, node)
        finally:
            events.senders -= 1               # the member's sending end is dropped here

    def _remove_cancelled(self):
        for group in range(len(self.live)):
            g = self.live[group]
            if g.phase == "Prefill" and g.members[g.leader].events.cancelled:
                replacement = next((mi for mi, m in enumerate(g.members) if m.live and not m.events.cancelled), None)
                if replacement is not None:
                    if g.pos > 0:
                        self.backend.seq_cp(g.members[g.leader].slot, g.members[replacement].slot, -1, -1)
                    g.leader = replacement
            cancelled = [mi for mi, m in enumerate(g.members) if m.live and m.events.cancelled]
            for mi in cancelled:
                self._finish_member(group, mi, "Cancelled")
        self._drop_dead_groups()

    def _rollback(self, kinds):
        for kind in kinds:
            group = kind[1]
            member = self.live[group].leader if kind[0] == "Prefill" else kind[2]
            m = self.live[group].members[member]
            try:
                self.backend.seq_rm(m.slot, -1, -1)
            except InferError:
                pass
            try:
                self.backend.request_free(m.request_id)
            except InferError:
                pass

    def _classify_step_error(self, error, needed):
        if error.kind == "Backend":
            try:
                mem = self.backend.memory()
                available = max(mem["cells_total"] - mem["cells_used"], 0)
                if needed > available:
                    return InferError("KvFull", needed=needed, available=available)
            except InferError:
                pass
        return error

    def _fail_all(self, error):
        to_release = []
        for g in self.live:
            for m in g.members:
                if m.live:
                    self._send_bounded(m.events, dict(type="Error", error=error.cloned()))
                    m.events.senders -= 1
                    m.live = False
                    to_release.append((m.slot, m.request_id))
        for slot, request_id in to_release:
            try:
                self.backend.seq_rm(slot, -1, -1)
            except InferError:
                pass
            try:
                self.backend.request_free(request_id)
            except InferError:
                pass
        self.live = []


def validate(r: Request):
    """request.rs:101-169"""
    import math
    if not r.prompt:
        raise invalid("a request requires a non-empty prompt")
    if not r.sampling:
        raise invalid("a request requires at least one sampling entry")
    if any(p.max_new_tokens == 0 for p in r.sampling):
        raise invalid("max_new_tokens must be greater than zero")
    if any((not math.isfinite(p.temperature)) or p.temperature <= 0.0 for p in r.sampling):
        raise invalid("temperature must be finite and greater than zero")
    if any(not (p.top_p > 0.0 and p.top_p <= 1.0) for p in r.sampling):
        raise invalid("top_p must be in (0, 1]")
    for p in r.sampling:
        if (not math.isfinite(p.min_p) or p.min_p < 0.0 or p.min_p > 1.0 or not math.isfinite(p.repeat_penalty)
                or p.repeat_penalty <= 0.0 or not math.isfinite(p.frequency_penalty)
                or not math.isfinite(p.presence_penalty) or any(not math.isfinite(b) for _, b in p.logit_bias)):
            raise invalid("min_p must be in [0, 1], repeat_penalty finite and > 0, frequency/presence penalties "
                          "and logit biases finite")
    if any(len(p.logit_bias) > 4096 for p in r.sampling):
        raise invalid("logit_bias takes at most 4096 entries")
    if any(s == "" for s in r.stop):
        raise invalid("stop strings must not be empty")
    if r.adapter is not None and r.adapter == "":
        raise invalid("an adapter name must not be empty")
    if r.retention is not None and r.retention[0] == "":
        raise invalid("a retention key must not be empty")


# ---- the synchronous batch driver (crates/retrograd-infer/src/sync.rs:96-149) -----------------------

def run_requests(scheduler: "Scheduler", requests, on_step=None):
    """Submits in order as the queue has room, pumps until all have ended, drains the streams after every
    step. Returns per request {"completions": [{tokens, logprobs, forced, text, finish}], "error"}."""
    pending = list(requests)
    streams, outcomes = [], []
    stalled = 0

    def absorb(outcome, e):
        if e["type"] == "Error":
            outcome["error"] = e["error"]
            return
        member = outcome["completions"][e["index"]]
        if e["type"] == "Token":
            member["tokens"].append(e["token"])
            member["logprobs"].append(e["logprob"])
            member["forced"].append(e.get("forced", False))
            member["text"] += e.get("text", "")
        else:
            member["finish"] = e["reason"]
            member["text"] += e.get("text", "")

    while True:
        while pending and scheduler.queued_len() < scheduler.queue_capacity():
            request = pending.pop(0)
            streams.append(scheduler.submit(request))
            outcomes.append({"completions": [dict(tokens=[], logprobs=[], forced=[], text="", finish=None)
                                             for _ in range(request.n())], "error": None})
        if not pending and scheduler.is_idle():
            break
        progressed = scheduler.pump()
        if on_step:
            on_step(scheduler)
        for stream, outcome in zip(streams, outcomes):
            for e in stream.drain():
                absorb(outcome, e)
        stalled = 0 if progressed else stalled + 1
        if stalled > 1024:
            raise InferError("Failed", "the scheduler made no progress with requests still queued")
    for stream, outcome in zip(streams, outcomes):
        for e in stream.drain():
            absorb(outcome, e)
    return outcomes
