"""The GBNF parser and matcher behind grammar-constrained sampling rows (retrograd_amd/csrc/grammar.hpp; the grammar
stage of reference crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:767-795, where the reference calls llama.cpp's
grammar sampler, absent from its checkout). Pinned from outside by the `regex` library: for grammars that are regular
the set of tokens allowed after a prefix must be exactly the tokens t for which prefix + t is a partial match of the
equivalent regular expression, and an end-of-generation token is allowed exactly when the prefix is a full match;
by hand-written prefix checkers for a grammar that is not regular; and by Python's json module for the built-in
JSON grammar. CPU only."""
import json
import random
import re
import subprocess
from pathlib import Path

import pytest
import regex

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def exe(tmp_path_factory):
    d = tmp_path_factory.mktemp("grammar_unit")
    out = d / "grammar_unit"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-o", str(out), str(ROOT / "tests/cpp/grammar_unit.cpp")], check=True)
    return out, d


def run(exe, lines):
    out, d = exe
    script = d / "script.txt"
    script.write_text("\n".join(lines) + "\n")
    r = subprocess.run([str(out), str(script)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    return r.stdout.splitlines()


def hx(s):
    b = s if isinstance(s, bytes) else s.encode()
    return b.hex() or "-"


class Session:
    """A scripted run: commands are queued with the check to apply to their output line."""

    def __init__(self, gbnf, tokens, eog=()):
        self.lines = ["token %s %d" % (hx(t), int(i in eog)) for i, t in enumerate(tokens)]
        self.lines.append("grammar " + hx(gbnf))
        self.checks = [lambda line: line == "ok" or pytest.fail(line)]

    def mask(self, want, note=""):
        self.lines.append("mask")
        w = " ".join(str(i) for i in sorted(want)) or "none"
        self.checks.append(lambda line, w=w, note=note: line == w or pytest.fail("allowed %s, want %s %s" % (line, w, note)))

    def accept(self, token, ok=True):
        self.lines.append("accept %d" % token)
        self.checks.append(lambda line, ok=ok: line == ("ok" if ok else "refused") or pytest.fail(line))

    def reset(self):
        self.lines.append("reset")
        self.checks.append(lambda line: line == "ok" or pytest.fail(line))

    def run(self, exe):
        got = run(exe, self.lines)
        assert len(got) == len(self.checks)
        for line, check in zip(got, self.checks):
            check(line)


REGULAR = [
    ('root ::= [a-c]+ ("x" | "yz")? [0-9]{2,3}', r'[a-c]+(x|yz)?[0-9]{2,3}',
     ["a", "b", "c", "ab", "x", "y", "z", "yz", "0", "7", "12", "345", "6789", "d", "a1", "cx", "xy", "bz"]),
    ('root ::= "ab"{2} c? d{1,} "."\nc ::= "c"   # a comment\nd ::= [d-f]', r'(ab){2}c?[d-f]+\.',
     ["a", "b", "ab", "abab", "ababc", "c", "d", "e", "f", "def", ".", "f.", "cd", "ba", "abc"]),
    ('root ::= ( "é" | [α-ω]+ |\n   "\\x41\\u00e9" ) "!"', r'(é|[α-ω]+|Aé)!', ["é", "α", "βγ", "ω!", "A", "Aé", "!", "é!", "a", "Aa"]),
    ('root ::= [^"\\\\]* "\\"" .', r'[^"\\]*".', ["a", '"', "\\", 'ab"', '"x', "xx", '""', "\n", 'a"\n']),
    ('root ::= item ("," item)*\nitem ::= [0-9]+ | "[" root "]"'.replace('"[" root "]"', '"n"'), r'([0-9]+|n)(,([0-9]+|n))*',
     ["1", "23", ",", "n", "n,", ",n", "1,2", ",,", "n1"]),
    ('root ::= "a"* "b"? "a"{0,2} "c"{3}', r'a*b?a{0,2}c{3}', ["a", "b", "c", "aa", "ab", "ba", "cc", "ccc", "bc", "ac", "baa", "baaa"]),
]


@pytest.mark.parametrize("case", range(len(REGULAR)))
def test_allowed_tokens_are_the_partial_matches_of_the_equivalent_regular_expression(exe, case):
    gbnf, pattern, tokens = REGULAR[case]
    tokens = tokens + ["<eos>"]
    eog = len(tokens) - 1
    rx = regex.compile(pattern, regex.DOTALL)
    rng = random.Random(case)
    s = Session(gbnf, tokens, eog={eog})
    for walk in range(40):
        prefix = ""
        for step in range(12):
            want = {i for i, t in enumerate(tokens[:-1]) if rx.fullmatch(prefix + t, partial=True)}
            if rx.fullmatch(prefix):
                want.add(eog)
            s.mask(want, "after %r" % prefix)
            wrong = [i for i in range(len(tokens)) if i not in want]
            if wrong:
                s.accept(rng.choice(wrong), ok=False)
            text = sorted(want - {eog})
            if not text:
                break
            t = rng.choice(text)
            s.accept(t)
            prefix += tokens[t]
        s.reset()
    s.run(exe)


def test_a_grammar_that_is_not_regular_counts_its_brackets(exe):
    tokens = ["(", ")", "a", "((", "))", "a)", "(a", ")(", "<eos>"]
    s = Session('root ::= "(" root ")" | "a"', tokens, eog={8})

    def state(prefix):          # depth still open and whether the "a" was seen; None if not a prefix of any sentence
        depth, seen = 0, False
        for ch in prefix:
            if ch == "(" and not seen:
                depth += 1
            elif ch == "a" and not seen:
                seen = True
            elif ch == ")" and seen and depth > 0:
                depth -= 1
            else:
                return None
        return depth, seen

    rng = random.Random(5)
    for walk in range(60):
        prefix = ""
        for step in range(14):
            want = {i for i, t in enumerate(tokens[:-1]) if state(prefix + t) is not None}
            if state(prefix) == (0, True):
                want.add(8)
            s.mask(want, "after %r" % prefix)
            text = sorted(want - {8})
            if not text:
                break
            t = rng.choice(text)
            s.accept(t)
            prefix += tokens[t]
        s.reset()
    s.run(exe)


def test_token_ids_and_text_split_inside_a_character(exe):
    # <[id]> takes the token whatever its text; !<[id]> any token but that one
    s = Session('root ::= <[3]> "a" !<[0]>', ["a", "b", "aa", "zzz", "<eos>"], eog={4})
    s.mask({3})
    s.accept(0, ok=False)
    s.accept(3)
    s.mask({0})
    s.accept(0)
    s.mask({1, 2, 3})               # any token but 0; an end-of-generation token only ever ends a complete sentence
    s.accept(2)
    s.mask({4})
    s.run(exe)
    # "é" is C3 A9: a byte token may stop inside it, and only the byte that finishes it may follow
    tokens = [b"\xc3", b"\xa9", "é", b"\xc3\xa9!", "!", b"\xce", b"\xa9!", "<eos>"]
    s = Session('root ::= "é" "!"', tokens, eog={7})
    s.mask({0, 2, 3})
    s.accept(5, ok=False)
    s.accept(0)
    s.mask({1, 6})
    s.accept(4, ok=False)
    s.accept(1)
    s.mask({4})
    s.accept(4)
    s.mask({7})
    s.accept(7)
    s.reset()
    s.accept(3)
    s.mask({7})
    s.run(exe)
    # a class decides on the possible completions: C3 can still become U+00C0..U+00FF, CE only U+0380..U+03BF
    s = Session('root ::= [à-ÿ] | [^\\x00-\\u03ff]', [b"\xc3", b"\xce", b"\xe4", "z", "é", "中"], eog=())
    s.mask({0, 2, 4, 5})
    s.run(exe)
    # lead bytes whose only ASCII completions would be overlong forms (C1 88 for "H") are no way to spell ASCII
    s = Session('root ::= "H" | "à"', [b"\xc1", b"\xe0", b"\xf0", b"\xc1\x88", "H", b"\xc3"], eog=())
    s.mask({4, 5})
    s.run(exe)


@pytest.mark.parametrize("gbnf, message", [
    ("root ::= missing", "undefined rule 'missing'"),
    ("start ::= \"a\"", "no 'root' rule"),
    ("root ::= root \"a\" | \"b\"", "left-recursive"),
    ("root ::= a \"x\"\na ::= b?\nb ::= root", "left-recursive"),
    ("root ::= \"abc", "unterminated literal"),
    ("root ::= [abc", "unterminated character class"),
    ("root ::= \"a\"\nroot ::= \"b\"", "defined twice"),
    ("root ::= \"a\"{3,2}", "run backwards"),
    ("root ::= (\"a\"", "')' is expected"),
    ("root ::= \"\\q\"", "unknown escape"),
    ("root = \"a\"", "'::=' is expected"),
    ("root ::= *", "end of the rule"),
    ("", "no 'root' rule"),
    ("root ::= \"abcdefghijkl\"{100000}", "too large"),
    ("root ::= " + "(" * 300 + "\"a\"" + ")" * 300, "nested too deeply"),
    # a chain of 5000 rules that each only name the next: as deep as it is long
    ("root ::= r0\n" + "".join("r%d ::= r%d\n" % (i, i + 1) for i in range(5000)) + "r5000 ::= \"a\"", "nested deeper"),
    # 2^14 ways to read the same text: the alternatives open at once are bounded
    ("root ::= x0\n" + "".join("x%d ::= \"a\" x%d \"b\" | \"a\" x%d \"c\"\n" % (i, i + 1, i + 1) for i in range(14)) + "x14 ::= \"!\"", None),
])
def test_invalid_grammars_are_refused_with_the_reason(exe, gbnf, message):
    if message is None:
        # valid, but walking "a" fourteen times doubles the open alternatives each time: an error, never a crash
        lines = run(exe, ["token 61 0", "grammar " + hx(gbnf)] + ["accept 0"] * 14)
        assert lines[0] == "ok"
        assert any(l.startswith("error: ") and "too ambiguous" in l for l in lines[1:]), lines
        return
    (line,) = run(exe, ["grammar " + hx(gbnf)])
    assert line.startswith("error: ") and message in line, line


def _json_grammar():
    text = (ROOT / "retrograd_amd/csrc/json_grammar.hpp").read_text()
    return text[text.index('R"GBNF(') + 7:text.index(')GBNF"')]


def _accepts(exe_, gbnf, alphabet, texts):
    """For each text whether the grammar takes every character and is complete at the end."""
    ids = {ch: i for i, ch in enumerate(alphabet)}
    lines = ["token %s 0" % hx(ch) for ch in alphabet] + ["token %s 1" % hx("<eos>"), "grammar " + hx(gbnf)]
    for t in texts:
        lines += ["accept %d" % ids[ch] for ch in t] + ["accept %d" % len(alphabet), "reset"]
    out = run(exe_, lines)[1:]
    res, at = [], 0
    for t in texts:
        n = len(t) + 1
        res.append(all(x == "ok" for x in out[at:at + n]))
        assert out[at + n] == "ok"
        at += n + 1
    return res


def test_the_built_in_json_grammar_against_the_json_module(exe):
    rng = random.Random(3)

    def value(depth):
        kind = rng.choice(["obj", "arr", "str", "num", "lit"] if depth < 3 else ["str", "num", "lit"])
        if kind == "obj":
            return {rng.choice(["a", "k\"q", "é", "x\\y", ""]): value(depth + 1) for _ in range(rng.randint(0, 3))}
        if kind == "arr":
            return [value(depth + 1) for _ in range(rng.randint(0, 3))]
        if kind == "str":
            return rng.choice(["", "text", "tab\there", "quote\"", "uni\u00e9\u4e2d", "back\\slash", "nl\n", "\x7f"])
        if kind == "num":
            return rng.choice([0, -0.0, 7, -12, 3.25, 1e10, -2.5e-3, 10 ** 20, 0.1])
        return rng.choice([True, False, None])

    good = []
    for i in range(60):
        doc = {"k%d" % j: value(0) for j in range(rng.randint(0, 3))}
        good.append(json.dumps(doc, ensure_ascii=bool(i % 2), indent=[None, 1][i % 3 == 0], separators=[(",", ":"), (", ", ": ")][i % 2]))
    texts = list(good)
    for g in good:                                   # damaged copies: one character dropped, doubled or replaced
        for _ in range(6):
            at = rng.randrange(len(g))
            how = rng.randrange(3)
            texts.append(g[:at] + (g[at + 1:] if how == 0 else g[at] + g[at:] if how == 1 else rng.choice('{}[]":,-+.eE019 \ttrufalsn\\/b\x01') + g[at + 1:]))
    texts += ['{"a":01}', '{"a":1.}', '{"a":.5}', '{"a":-}', '{"a":1e}', '{"a":"\\x"}', '{"a":"\\u12g4"}', '{"a":"\x01"}', '[1]', '"s"',
              '{"a":1,}', '{,}', '{"a" 1}', '{"a":tru}', '{"a":[1,]}', '{"a":1} ', '{ }', '{"a":\t[ ]\n}', ' {}', '{"a":NaN}', '{"a":1}{}']
    alphabet = sorted(set("".join(texts)))
    got = _accepts(exe, _json_grammar(), alphabet, texts)

    def is_object(t):
        if t[:1] != "{":                             # the grammar starts at the brace; json.loads would skip white space
            return False
        try:
            return isinstance(json.loads(t, parse_constant=lambda c: (_ for _ in ()).throw(ValueError(c))), dict)
        except (ValueError, RecursionError):
            return False

    want = [is_object(t) for t in texts]
    wrong = [(t, g, w) for t, g, w in zip(texts, got, want) if g != w]
    assert not wrong, wrong[:5]
    assert sum(want) >= 60 and want.count(False) >= 100


# ---- JSON schema -> GBNF (retrograd_amd/csrc/json_schema.hpp, behind retro_grammar_from_json_schema) -------------
# The reference converts with llama.cpp's json_schema_to_grammar, absent from its checkout, and its tests only
# require that constrained output parses and fits the schema (tests/judge_local.rs:82-130). The converter here is
# checked the same way, exhaustively where that one samples: for each schema a validator written in Python decides
# which of many instances (generated, then damaged) fit, and the grammar made from the schema must accept exactly
# those. The language llama.cpp's converter would give for the same schema is not pinned (white space, the order
# of members): parity with it is unpinned.

SCHEMAS = [
    {"type": "object", "properties": {"name": {"type": "string"}, "age": {"type": "integer"},
                                      "tags": {"type": "array", "items": {"type": "string"}, "maxItems": 3},
                                      "kind": {"enum": ["a", "b", 3, None]}}, "required": ["name", "tags"]},
    {"$defs": {"node": {"type": "object", "properties": {"v": {"type": "number"}, "kids": {"type": "array", "items": {"$ref": "#/$defs/node"}}},
                        "required": ["v"]}}, "$ref": "#/$defs/node"},
    {"type": "object", "properties": {"x": {"anyOf": [{"type": "boolean"}, {"const": "none"}]}, "y": {"type": ["integer", "null"]}},
     "required": ["x", "y"]},
    {"type": "object", "properties": {"id": {"type": "integer"}}, "required": ["id"], "additionalProperties": {"type": "string"}},
    {"type": "object"},
    {"type": "array", "prefixItems": [{"type": "string"}, {"type": "integer"}]},
    {"type": "string", "minLength": 2, "maxLength": 4},
    {"type": "array", "items": {"type": "integer"}, "minItems": 2, "maxItems": 3},
    {"type": "object", "properties": {"a": {"type": "boolean"}, "b": {"type": "null"}, "c": {}}, "additionalProperties": False},
    {"type": "object", "properties": {"q": {"type": "string"}}, "additionalProperties": True},
    # further members must not bear a declared name, however close theirs comes to one
    {"type": "object", "properties": {"q": {"type": "string"}, "qu\"x": {"type": "null"}, "é": {}, "t\tab": {"type": "boolean"}},
     "additionalProperties": {"type": "integer"}},
]


def _fits(schema, v, root):
    if schema is True or schema == {}:
        return True
    if "$ref" in schema:
        node = root
        for part in schema["$ref"][2:].split("/"):
            node = node[part]
        return _fits(node, v, root)
    if "const" in schema:
        return type(v) is type(schema["const"]) and v == schema["const"]
    if "enum" in schema:
        return any(type(v) is type(e) and v == e for e in schema["enum"])
    for key in ("anyOf", "oneOf"):
        if key in schema:
            return any(_fits(s, v, root) for s in schema[key])
    t = schema.get("type")
    if isinstance(t, list):
        return any(_fits(dict(schema, type=one), v, root) for one in t)
    if t is None:
        t = "object" if "properties" in schema else None
    if t == "object":
        if not isinstance(v, dict):
            return False
        props = schema.get("properties", {})
        extra = schema.get("additionalProperties")
        if not props and extra in (None, True):
            return True
        keys = list(v)
        declared = [k for k in keys if k in props]
        others = [k for k in keys if k not in props]
        if keys != declared + others or declared != [k for k in props if k in v]:
            return False                                     # declared members in the schema's order, the others after
        if any(k not in v for k in schema.get("required", [])):
            return False
        if others and extra in (None, False):
            return False
        return all(_fits(props[k], v[k], root) for k in declared) and \
            all(extra is True or _fits(extra, v[k], root) for k in others)
    if t == "array":
        if not isinstance(v, list):
            return False
        if "prefixItems" in schema:
            return len(v) == len(schema["prefixItems"]) and all(_fits(s, x, root) for s, x in zip(schema["prefixItems"], v))
        if len(v) < schema.get("minItems", 0) or len(v) > schema.get("maxItems", 1 << 30):
            return False
        return all(_fits(schema.get("items", True), x, root) for x in v)
    if t == "string":
        return isinstance(v, str) and schema.get("minLength", 0) <= len(v) <= schema.get("maxLength", 1 << 30)
    if t == "integer":
        return isinstance(v, int) and not isinstance(v, bool)
    if t == "number":
        return isinstance(v, (int, float)) and not isinstance(v, bool)
    if t == "boolean":
        return isinstance(v, bool)
    if t == "null":
        return v is None
    raise AssertionError(schema)


def _instance(schema, root, rng, depth=0):
    if schema is True or schema == {}:
        return rng.choice([1, "s", None, True, [1, "x"], {"k": 2.5}])
    if "$ref" in schema:
        node = root
        for part in schema["$ref"][2:].split("/"):
            node = node[part]
        return _instance(node, root, rng, depth + 1)
    if "const" in schema:
        return schema["const"]
    if "enum" in schema:
        return rng.choice(schema["enum"])
    for key in ("anyOf", "oneOf"):
        if key in schema:
            return _instance(rng.choice(schema[key]), root, rng, depth)
    t = schema.get("type")
    if isinstance(t, list):
        t = rng.choice(t)
    if t == "object" or (t is None and "properties" in schema):
        out = {}
        for k, s in schema.get("properties", {}).items():
            if k in schema.get("required", []) or rng.random() < 0.5:
                out[k] = _instance(s, root, rng, depth + 1)
        extra = schema.get("additionalProperties")
        if extra not in (None, False) or not schema.get("properties"):
            for k in rng.sample(["extra0", "extra1", "qu", "", "qq", "qu\"", "qu\"xy", "éé", "e\n", "t", "t\t", "t\tabs", "\\"], rng.randint(0, 3)):
                out[k] = _instance(True if extra in (None, True) else extra, root, rng, depth + 1)
        return out
    if t == "array":
        if "prefixItems" in schema:
            return [_instance(s, root, rng, depth + 1) for s in schema["prefixItems"]]
        lo, hi = schema.get("minItems", 0), schema.get("maxItems", 3)
        n = rng.randint(lo, hi) if depth < 3 else lo
        return [_instance(schema.get("items", True), root, rng, depth + 1) for _ in range(n)]
    if t == "string":
        n = rng.randint(schema.get("minLength", 0), schema.get("maxLength", 5))
        return "".join(rng.choice("ab \"\\é") for _ in range(n))
    if t == "integer":
        return rng.choice([0, 7, -12, 100])
    if t == "number":
        return rng.choice([0, 1.5, -2, 1e-5, 3e20])
    if t == "boolean":
        return rng.random() < 0.5
    if t == "null":
        return None
    raise AssertionError(schema)


def _damage(v, rng):
    """A nearby value: a member dropped, added, moved or retyped; an item added or dropped."""
    v = json.loads(json.dumps(v))
    spots = []

    def walk(x, path):
        spots.append(path)
        if isinstance(x, dict):
            for k in x:
                walk(x[k], path + [k])
        elif isinstance(x, list):
            for i, y in enumerate(x):
                walk(y, path + [i])
    walk(v, [])
    path = rng.choice(spots)
    other = rng.choice([0, "zz", None, True, 2.5, [], {}, [1, 2, 3, 4], "a", "abcde"])
    if not path:
        if isinstance(v, dict) and v and rng.random() < 0.7:
            k = rng.choice(list(v))
            how = rng.randrange(3)
            if how == 0:
                del v[k]
            elif how == 1:
                v = dict(list(v.items())[::-1])
            else:
                v["zzz"] = other
            return v
        if isinstance(v, list) and rng.random() < 0.7:
            return v + [other] if rng.random() < 0.5 or not v else v[:-1]
        return other
    parent = v
    for p in path[:-1]:
        parent = parent[p]
    parent[path[-1]] = other
    return v


def _gbnf_of(exe, schema):
    out, d = exe
    unit = d / "schema_unit"
    if not unit.exists():
        subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-o", str(unit), str(ROOT / "tests/cpp/schema_unit.cpp")], check=True)
    f = d / "schema.json"
    f.write_text(json.dumps(schema))
    r = subprocess.run([str(unit), str(f)], capture_output=True, text=True, timeout=60)
    return r.returncode, r.stdout


@pytest.mark.parametrize("index", range(len(SCHEMAS)))
def test_a_schemas_grammar_accepts_exactly_the_instances_that_fit(exe, index):
    schema = SCHEMAS[index]
    code, gbnf = _gbnf_of(exe, schema)
    assert code == 0, gbnf
    rng = random.Random(100 + index)
    values = [_instance(schema, schema, rng) for _ in range(40)]
    values += [_damage(v, rng) for v in values for _ in range(4)]
    texts, want = [], []
    for i, v in enumerate(values):
        texts.append(json.dumps(v, ensure_ascii=False, separators=[(",", ":"), (", ", ": ")][i % 2]))
        want.append(_fits(schema, v, schema))
    assert all(want[:40]) and want.count(False) >= 20, (want.count(True), want.count(False))
    got = _accepts(exe, gbnf, sorted(set("".join(texts))), texts)
    wrong = [(t, g, w) for t, g, w in zip(texts, got, want) if g != w]
    assert not wrong, wrong[:5]


@pytest.mark.parametrize("schema, message", [
    ({"type": "string", "pattern": "^a+$"}, "'pattern'"),
    ({"type": "integer", "minimum": 0}, "'minimum'"),
    ({"allOf": [{"type": "string"}]}, "'allOf'"),
    ({"$ref": "http://example.com/x.json"}, "$ref"),
    ({"$ref": "#/$defs/missing"}, "points at nothing"),
    ({"type": "object", "properties": {"a": {}}, "required": ["b"]}, "'b'"),
    ({"type": "frob"}, "unknown JSON schema type"),
])
def test_schemas_outside_the_subset_are_refused_with_the_keyword(exe, schema, message):
    code, out = _gbnf_of(exe, schema)
    assert code == 1 and out.startswith("error: ") and message in out, out
