"""Generates the tokenizer fixtures: a small byte-fallback BPE model trained with SentencePiece in
this container (LLaMA's tokenizer settings: BPE, byte fallback, identity normalisation, dummy prefix,
digits split, ids unk 0 / bos 1 / eos 2 / bytes 3..258), written as a vocab file in the reference's
format (extract.py:45-61: int32 count, count x {int32 offset, float score}, NUL-terminated pieces with
U+2581 replaced by a space), and SentencePiece's own encodings of the test strings.

    python tests/golden/make_tokenizer_fixture.py

Writes tests/golden/spm_bpe.model, tests/golden/spm_bpe_vocab.bin and tests/golden/spm_bpe_cases.json.
"""
import io
import json
import os
import random
import struct

import sentencepiece as spm

HERE = os.path.dirname(os.path.abspath(__file__))

WORDS = ("the of and to in a is that for it as was with be by on not he this are or his from at which but have an "
         "had they you were their one all we can her has there been if more when will would who so no out up into "
         "model token weight matrix layer vector cache memory kernel thread wave block scale code row column "
         "building website easy steps first second third choose domain name design content publish test "
         "number value compute result input output attention softmax rotary normal quantise round half float").split()


def corpus():
    rng = random.Random(0)
    lines = []
    for _ in range(4000):
        n = rng.randint(3, 14)
        words = [rng.choice(WORDS) for _ in range(n)]
        if rng.random() < 0.3:
            words.insert(rng.randrange(len(words)), str(rng.randint(0, 9999)))
        line = " ".join(words)
        if rng.random() < 0.5:
            line = line.capitalize() + rng.choice(".?!:")
        lines.append(line)
    return lines


CASES = [
    "Building a website can be done in 10 easy steps:",
    "the model",
    "a",
    "attention is all you need",
    "Hello, world!",
    "1234567890",
    "tokenweightmatrix",
    "the  model with  two spaces",
    "café naïve über",
    "你喗 世界",
    "emoji \U0001f600 end",
    "tab\there",
    "UPPER lower MiXeD",
    "x" * 40,
    "the the the the the the",
    "quantise the weight matrix by block, then round half away from zero.",
]


def main():
    model = io.BytesIO()
    spm.SentencePieceTrainer.train(
        sentence_iterator=iter(corpus()), model_writer=model, vocab_size=640, model_type="bpe", byte_fallback=True,
        character_coverage=1.0, normalization_rule_name="identity", add_dummy_prefix=True,
        remove_extra_whitespaces=False, split_digits=True, unk_id=0, bos_id=1, eos_id=2, pad_id=-1,
        num_threads=1, minloglevel=2)
    with open(os.path.join(HERE, "spm_bpe.model"), "wb") as f:   # input of the vocabulary extractor's test
        f.write(model.getvalue())
    sp = spm.SentencePieceProcessor(model_proto=model.getvalue())
    n = sp.vocab_size()
    pieces = [sp.id_to_piece(i).replace("▁", " ").encode("utf-8") for i in range(n)]
    assert sp.id_to_piece(3) == "<0x00>" and sp.id_to_piece(258) == "<0xFF>"
    offset = 4 + 8 * n
    with open(os.path.join(HERE, "spm_bpe_vocab.bin"), "wb") as f:
        f.write(struct.pack("<i", n))
        for i, piece in enumerate(pieces):
            f.write(struct.pack("<if", offset, sp.get_score(i)))
            offset += len(piece) + 1
        for piece in pieces:
            f.write(piece + b"\0")
    cases = [{"text": t, "ids": sp.encode(t)} for t in CASES]
    with open(os.path.join(HERE, "spm_bpe_cases.json"), "w") as f:
        json.dump({"sentencepiece": spm.__version__, "vocab_size": n, "cases": cases}, f, indent=1, ensure_ascii=True)
    print("vocab %d pieces; %d cases" % (n, len(cases)))


if __name__ == "__main__":
    main()
