"""Text -> token ids for sentencepiece-kind vocabularies (retrograd_amd/csrc/tokenizer.hpp; the host side of
retro_engine_tokenize*, reference crates/retrograd-ffi/runtime/src/retro_engine.cpp:331-378) against the ids of the
sentencepiece library itself, committed as tests/golden/spm_reference_ids.json by tests/golden/spm_reference_ids.py.
The reference hands the text to llama.cpp's tokenizer (absent from its checkout) and its tests hold no tokenisation
vectors; llama.cpp's SPM tokenizer reproduces sentencepiece's BPE model, which is what pins this one. CPU only."""
import json
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
GOLDEN = json.loads((ROOT / "tests/golden/spm_reference_ids.json").read_text())


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    d = tmp_path_factory.mktemp("tokenizer_unit")
    exe = d / "tokenizer_unit"
    subprocess.run(["g++", "-std=c++17", "-O1", "-o", str(exe), str(ROOT / "tests/cpp/tokenizer_unit.cpp")], check=True)
    vocab = d / "vocab.txt"
    vocab.write_text("".join("%s %r %d\n" % (p.encode().hex() or "-", s, t) for p, s, t in GOLDEN["vocab"]))
    return exe, vocab, d


def _run(harness, cases, add_eos=False):
    exe, vocab, d = harness
    texts = d / "texts.txt"
    texts.write_text("".join("%d %d %s\n" % (a, p, t.encode().hex() or "-") for a, p, t in cases))
    r = subprocess.run([str(exe), str(vocab), str(texts), str(GOLDEN["bos"]), str(GOLDEN["eos"]), "1" if add_eos else "0"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    return [[int(x) for x in line.split()] for line in r.stdout.splitlines()]


def test_ids_equal_the_sentencepiece_librarys(harness):
    got = _run(harness, [(0, 0, c["text"]) for c in GOLDEN["cases"]])
    for c, ids in zip(GOLDEN["cases"], got):
        assert ids == c["ids"], c["text"]
    # the cases reach the byte fallback, doubled spaces and multi-byte characters
    byte_ids = {i for i, (_, _, t) in enumerate(GOLDEN["vocab"]) if t == 6}
    assert any(byte_ids & set(c["ids"]) for c in GOLDEN["cases"])


def test_special_tokens_and_the_flags(harness):
    bos, eos = GOLDEN["bos"], GOLDEN["eos"]
    plain = {c["text"]: c["ids"] for c in GOLDEN["cases"]}
    (with_bos,), (with_both,) = _run(harness, [(1, 0, "hello world")]), _run(harness, [(1, 0, "hello world")], add_eos=True)
    assert with_bos == [bos] + plain["hello world"]
    assert with_both == [bos] + plain["hello world"] + [eos]
    # parse_special reads the text of a control token as the token; the text after it starts a new stretch
    # (a space in front, as at the start of the text); without it the same characters are ordinary text
    (parsed,), (literal,) = _run(harness, [(0, 1, "<s>hello world</s>")]), _run(harness, [(0, 0, "<s>hello world</s>")])
    assert parsed == [bos] + plain["hello world"] + [eos]
    assert literal != parsed and bos not in literal
    (mixed,) = _run(harness, [(0, 1, "mixed <s> inside")])
    assert mixed.count(bos) == 1 and mixed != plain["mixed <s> inside"]
    (empty,) = _run(harness, [(1, 1, "")]) or ([],)
    assert empty in ([bos], [])
