"""Writes tests/golden/bpe_reference_ids.json: for each pre-tokeniser pattern the product builds (the ones GGUF files
name "llama-bpe", "qwen2" and "gpt-2" in tokenizer.ggml.pre) a small byte-level byte-pair vocabulary trained by the
Hugging Face `tokenizers` library on a synthetic corpus, and that library's own words (the pre-tokeniser's pieces)
and ids for a list of texts. tests/test_tokenizer.py requires the product's tokenizer to reproduce both.

The patterns are the published ones of the Llama 3, Qwen 2 and GPT-2 tokenizer.json files.

Run in the build container (tokenizers 0.22 is importable there):  python tests/golden/bpe_reference_ids.py"""
import json
import random
import sys
from pathlib import Path

OUT = Path(__file__).resolve().parent / "bpe_reference_ids.json"

LLAMA3 = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+"
          r"|\s+(?!\S)|\s+")
QWEN2 = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+"
         r"|\s+(?!\S)|\s+")

WORDS = ["the", "quick", "brown", "fox", "jumps", "over", "lazy", "dog", "Hello", "world", "token", "model", "llama",
         "über", "naïve", "straße", "日本語", "テスト", "data", "quantum", "attention", "is", "all", "you", "need", "2024",
         "3.14159", "don't", "I'll", "we've", "re-use", "e-mail", "x=y+z;", "{json:", "\"key\"}", "C++", "#include",
         "snake_case", "CamelCase", "1234567", "\n", "\n\n", "  ", "...", "!?"]

TEXTS = [
    "Hello world",
    " Hello  world ",
    "The quick brown fox jumps over the lazy dog.",
    "don't I'll we've they'RE HE'S it'D y'all 'tis",
    "1 12 123 1234 12345 1234567 3.14159 2024-11-25 ①②③ ४५६",
    "über naïve straße 日本語のテスト Ελληνικά",
    "emoji \U0001f642\U0001f680 done",
    "tabs\tand\nnewlines\r\n\r\n  indented\n\n\nend",
    "trailing spaces   ",
    "   leading spaces and   runs   of   them",
    "x=y+z; {json: \"key\"} C++ #include <stdio.h>\n// comment!!!\n",
    "punct...\n\nthen, (parens) [brackets] -- dashes --\r\nwindows",
    "no break em space　ideographic",
    "a",
    " ",
    "\n",
    "zzzzzzzzzzzzzzzzzzzzzzzz",
    "the the the quick quick",
    "<|begin_of_text|>literal text of a control token<|end_of_text|>",
]


def build(kind):
    from tokenizers import Regex, Tokenizer, decoders, models, pre_tokenizers, trainers
    tok = Tokenizer(models.BPE(ignore_merges=kind == "llama-bpe"))
    if kind == "gpt-2":
        split = None
        tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=True)
    else:
        split = pre_tokenizers.Split(Regex(LLAMA3 if kind == "llama-bpe" else QWEN2), behavior="isolated", invert=False)
        tok.pre_tokenizer = pre_tokenizers.Sequence([split, pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    tok.decoder = decoders.ByteLevel()
    rng = random.Random(11)
    corpus = [" ".join(rng.choice(WORDS) for _ in range(rng.randint(4, 16))) for _ in range(4000)]
    trainer = trainers.BpeTrainer(vocab_size=640, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), show_progress=False,
                                  special_tokens=["<|begin_of_text|>", "<|end_of_text|>"])
    tok.train_from_iterator(corpus, trainer)
    spec = json.loads(tok.to_str())
    by_id = sorted(spec["model"]["vocab"].items(), key=lambda kv: kv[1])
    assert [i for _, i in by_id] == list(range(len(by_id)))
    merges = [m if isinstance(m, str) else " ".join(m) for m in spec["model"]["merges"]]
    cases = []
    for text in TEXTS:
        words = [text[a:b] for _, (a, b) in tok.pre_tokenizer.pre_tokenize_str(text)]
        enc = tok.encode(text, add_special_tokens=False)
        assert tok.decode(enc.ids, skip_special_tokens=False) == text
        cases.append({"text": text, "words": words, "ids": enc.ids})
    return {"pre": kind, "tokens": [t for t, _ in by_id], "control": [0, 1], "merges": merges, "cases": cases}


def main() -> int:
    import tokenizers
    out = {"tokenizers": tokenizers.__version__, "kinds": [build(k) for k in ("llama-bpe", "qwen2", "gpt-2")]}
    OUT.write_text(json.dumps(out, ensure_ascii=True, indent=0))
    print("wrote", OUT, [(k["pre"], len(k["tokens"]), len(k["merges"])) for k in out["kinds"]])
    return 0


if __name__ == "__main__":
    sys.exit(main())
