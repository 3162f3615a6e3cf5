"""Text -> token ids (retrograd_amd/csrc/tokenizer.hpp; the host side of retro_engine_tokenize*, reference
crates/retrograd-ffi/runtime/src/retro_engine.cpp:331-378) against the ids of the libraries that define the two
vocabulary kinds: sentencepiece for tokenizer.ggml.model = "llama" (tests/golden/spm_reference_ids.json, written by
tests/golden/spm_reference_ids.py) and Hugging Face tokenizers for the byte-level byte-pair kind "gpt2" with the
Llama 3, Qwen 2 and GPT-2 pre-tokeniser patterns (tests/golden/bpe_reference_ids.json, by bpe_reference_ids.py).
The reference hands the text to llama.cpp's tokenizer (absent from its checkout) and its tests hold no tokenisation
vectors; llama.cpp's tokenizers reproduce those two libraries, which is what pins this one. CPU only."""
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
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-o", str(exe), str(ROOT / "tests/cpp/tokenizer_unit.cpp")], check=True)
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


# ---- byte-pair vocabularies ----

BPE = json.loads((ROOT / "tests/golden/bpe_reference_ids.json").read_text())


def _run_bpe(harness, kind, cases, what):
    exe, _, d = harness
    vocab, merges, texts = d / ("bpe-%s-vocab.txt" % kind["pre"]), d / ("bpe-%s-merges.txt" % kind["pre"]), d / "bpe-texts.txt"
    vocab.write_text("".join("%s 0 %d\n" % (t.encode().hex(), 3 if i in kind["control"] else 1)
                             for i, t in enumerate(kind["tokens"])))
    merges.write_text("".join(m.encode().hex() + "\n" for m in kind["merges"]))
    texts.write_text("".join("%d %d %s\n" % (a, p, t.encode().hex() or "-") for a, p, t in cases))
    r = subprocess.run([str(exe), str(vocab), str(texts), "0", "1", "0", kind["pre"], str(merges), what],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    lines = r.stdout.splitlines()
    return lines[0], lines[1:]


@pytest.mark.parametrize("kind", BPE["kinds"], ids=[k["pre"] for k in BPE["kinds"]])
def test_words_equal_the_tokenizers_librarys_pre_tokeniser(harness, kind):
    _, got = _run_bpe(harness, kind, [(0, 0, c["text"]) for c in kind["cases"]], "words")
    for c, line in zip(kind["cases"], got):
        assert [bytes.fromhex(w).decode() for w in line.split()] == c["words"], c["text"]


@pytest.mark.parametrize("kind", BPE["kinds"], ids=[k["pre"] for k in BPE["kinds"]])
def test_ids_equal_the_tokenizers_librarys(harness, kind):
    # the library always reads the text of an added token as that token: such a case runs with parse_special
    first, got = _run_bpe(harness, kind, [(0, int("<|" in c["text"]), c["text"]) for c in kind["cases"]], "ids")
    assert first == "add_bos %d" % (kind["pre"] == "llama-bpe")         # only the Llama 3 kind opens with BOS by default
    for c, line in zip(kind["cases"], got):
        assert [int(x) for x in line.split()] == c["ids"], c["text"]
    # merges happened (fewer ids than bytes) and, under ignore_merges, whole words were taken
    assert any(len(c["ids"]) < len(c["text"].encode()) // 2 for c in kind["cases"])
    # parse_special: the text of a control token is that token, and what follows is split on its own
    text = "<|begin_of_text|>Hello world<|end_of_text|>"
    plain = next(c["ids"] for c in kind["cases"] if c["text"] == "Hello world")
    _, (parsed, literal) = _run_bpe(harness, kind, [(0, 1, text), (0, 0, text)], "ids")
    assert [int(x) for x in parsed.split()] == [0] + plain + [1]
    assert 0 not in [int(x) for x in literal.split()]


@pytest.mark.parametrize("alias,of", [("lfm2", "llama-bpe"), ("pixtral", "llama-bpe"), ("falcon-h1", "llama-bpe"), ("midm-2.0", "llama-bpe"),
                                      ("llama3", "llama-bpe"), ("phi-2", "gpt-2"), ("deepseek-r1-qwen", "qwen2")])
def test_pattern_names_that_llama_cpp_maps_to_one_pattern_tokenize_alike(harness, alias, of):
    # llama.cpp's vocabulary loader gives several tokenizer.ggml.pre names the same pattern and defaults
    # (llama-vocab.cpp); the reference's own CPU fixture model names "lfm2". Same words, same ids, same BOS default.
    kind = next(k for k in BPE["kinds"] if k["pre"] == of)
    cases = [(0, int("<|" in c["text"]), c["text"]) for c in kind["cases"]]
    first, want = _run_bpe(harness, kind, cases, "ids")
    again, got = _run_bpe(harness, dict(kind, pre=alias), cases, "ids")
    assert again == first and got == want


def test_an_unknown_pattern_is_refused(harness):
    exe, _, d = harness
    kind = dict(BPE["kinds"][0], pre="some-other-pattern")
    vocab, merges, texts = d / "x-vocab.txt", d / "x-merges.txt", d / "x-texts.txt"
    vocab.write_text("61 0 1\n")
    merges.write_text("")
    texts.write_text("0 0 61\n")
    r = subprocess.run([str(exe), str(vocab), str(texts), "0", "1", "0", kind["pre"], str(merges), "ids"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "some-other-pattern" in r.stdout and "not built" in r.stdout


def test_byte_pieces_that_are_not_two_hex_digits_stand_for_no_byte(harness):
    # A malformed vocabulary: BYTE-type pieces "<0x-1>", "<0xZZ>", "<0x+7>", "<0x 1>" must neither index the byte
    # table out of bounds nor throw (the harness runs under the address and undefined-behaviour sanitizers); the
    # ids of the well-formed vocabulary in front of them do not change.
    exe, vocab, d = harness
    bad = d / "vocab_bad.txt"
    extra = ["<0x-1>", "<0xZZ>", "<0x+7>", "<0x 1>"]
    bad.write_text(vocab.read_text() + "".join("%s 0.0 6\n" % p.encode().hex() for p in extra))
    case = GOLDEN["cases"][0]
    texts = d / "texts_bad.txt"
    texts.write_text("0 0 %s\n" % (case["text"].encode().hex() or "-"))
    r = subprocess.run([str(exe), str(bad), str(texts), str(GOLDEN["bos"]), str(GOLDEN["eos"]), "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert [int(x) for x in r.stdout.split()] == case["ids"]
