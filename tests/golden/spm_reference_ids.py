"""Writes tests/golden/spm_reference_ids.json: a small sentencepiece BPE vocabulary (byte fallback, dummy prefix,
identity normalisation - the settings of the Llama-family tokenizer models that GGUF files carry as
tokenizer.ggml.model = "llama") trained on a synthetic corpus, and the ids the sentencepiece library itself gives
for a list of texts. tests/test_tokenizer.py requires the product's tokenizer to reproduce them.

Run in the build container (sentencepiece 0.2 is importable there):  python tests/golden/spm_reference_ids.py"""
import io
import json
import os
import random
import sys
from pathlib import Path

OUT = Path(__file__).resolve().parent / "spm_reference_ids.json"

WORDS = ["the", "quick", "brown", "fox", "jumps", "over", "lazy", "dog", "hello", "world", "token", "model", "llama",
         "über", "naïve", "straße", "日本語", "テスト", "data", "quantum", "attention", "is", "all", "you", "need", "2024",
         "3.14159", "don't", "re-use", "e-mail", "x=y+z;", "{json:", "\"key\"}", "C++", "#include", "snake_case", "CamelCase"]

TEXTS = [
    "hello world",
    " hello  world ",                       # leading, doubled and trailing spaces
    "The quick brown fox jumps over the lazy dog.",
    "über naïve straße",
    "日本語のテスト",
    "emoji \U0001f642 and an unseen script: Ελληνικά",      # byte fallback
    "tabs\tand\nnewlines\r\n",
    "attention is all you need 2024 3.14159",
    "x=y+z; {json: \"key\"} C++ #include snake_case CamelCase",
    "a",
    "zzzzzzzzzzzzzzzzzzzzzzzz",
    "<s>literal text of a control token</s>",
    "mixed <s> inside",
]


def main() -> int:
    import sentencepiece as spm
    rng = random.Random(7)
    corpus = [" ".join(rng.choice(WORDS) for _ in range(rng.randint(4, 16))) for _ in range(6000)]
    model = io.BytesIO()
    devnull = os.open(os.devnull, os.O_WRONLY)
    saved = os.dup(2)
    os.dup2(devnull, 2)                      # the trainer logs a page per call
    try:
        spm.SentencePieceTrainer.train(sentence_iterator=iter(corpus), model_writer=model, vocab_size=560, model_type="bpe",
                                       byte_fallback=True, character_coverage=0.9995, normalization_rule_name="identity",
                                       add_dummy_prefix=True, remove_extra_whitespaces=False, split_digits=True,
                                       num_threads=1)
    finally:
        os.dup2(saved, 2)
    sp = spm.SentencePieceProcessor(model_proto=model.getvalue())
    vocab = []
    for i in range(sp.get_piece_size()):
        t = 6 if sp.is_byte(i) else 3 if sp.is_control(i) else 2 if sp.is_unknown(i) else 5 if sp.is_unused(i) else 1
        vocab.append([sp.id_to_piece(i), sp.get_score(i), t])
    cases = []
    for text in TEXTS:
        # sentencepiece never reads the text of a control token as that token: these are the ids of plain text
        cases.append({"text": text, "ids": sp.encode(text)})
    OUT.write_text(json.dumps({"sentencepiece": spm.__version__, "bos": sp.bos_id(), "eos": sp.eos_id(), "unk": sp.unk_id(),
                               "vocab": vocab, "cases": cases}, ensure_ascii=True, indent=0))
    print("wrote", OUT, len(vocab), "pieces,", len(cases), "cases")
    return 0


if __name__ == "__main__":
    sys.exit(main())
