"""Vocabulary reader and tokenizer (host code, no GPU): the C handles against the plain-Python
oracle, and both against SentencePiece's own output on a BPE model trained in the build container
(tests/golden/make_tokenizer_fixture.py)."""
import json
import os
import struct
import sys

import numpy as np
import pytest

import lcu

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle"))
import tokenizer_oracle as T  # noqa: E402

P = lcu.package()
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
VOCAB = os.path.join(GOLDEN, "spm_bpe_vocab.bin")


@pytest.fixture(scope="module")
def spm_cases():
    return json.load(open(os.path.join(GOLDEN, "spm_bpe_cases.json")))


@pytest.fixture(scope="module")
def oracle_vocab():
    return T.read_vocab(open(VOCAB, "rb").read())


@pytest.fixture(scope="module")
def vocab():
    v = P.Vocabulary(VOCAB)
    yield v
    v.close()


def write_vocab(path, entries):
    """entries: list of (bytes piece, float score) for ids 0.. in the reference's file format"""
    n = len(entries)
    offset = 4 + 8 * n
    with open(path, "wb") as f:
        f.write(struct.pack("<i", n))
        for piece, score in entries:
            f.write(struct.pack("<if", offset, score))
            offset += len(piece) + 1
        for piece, _ in entries:
            f.write(piece + b"\0")


def base_entries():
    e = [(b"<unk>", 0.0), (b"<s>", 0.0), (b"</s>", 0.0)]
    e += [(b"<0x%02X>" % i, 0.0) for i in range(256)]
    return e


def test_oracle_matches_sentencepiece(spm_cases, oracle_vocab):
    assert spm_cases["vocab_size"] == len(oracle_vocab[0])
    for case in spm_cases["cases"]:
        assert T.tokenize(case["text"].encode(), False, *oracle_vocab) == case["ids"], case["text"]
        assert T.tokenize(case["text"].encode(), True, *oracle_vocab) == [1] + case["ids"]


def test_library_matches_sentencepiece(spm_cases, vocab):
    assert len(vocab) == spm_cases["vocab_size"]
    for case in spm_cases["cases"]:
        assert vocab.tokenize(case["text"], bos=False) == case["ids"], case["text"]
        assert vocab.tokenize(case["text"], bos=True) == [1] + case["ids"]


def test_library_matches_oracle_on_random_text(vocab, oracle_vocab):
    pieces = oracle_vocab[0]
    rng = np.random.default_rng(0)
    words = [p for p in pieces[259:] if p.strip()]
    for trial in range(300):
        kind = trial % 3
        if kind == 0:    # words of the vocabulary glued with and without spaces
            text = b"".join(words[i] + (b" " if rng.random() < 0.3 else b"") for i in rng.integers(0, len(words), 12))
        elif kind == 1:  # arbitrary bytes, invalid UTF-8 included (no NUL: C strings end there in the file format)
            text = bytes(rng.integers(1, 256, int(rng.integers(1, 40))).astype(np.uint8))
        else:            # text that starts with a space gets no second one (llama_cu.cu:1353)
            text = b" " + words[int(rng.integers(0, len(words)))] + b"  " + words[int(rng.integers(0, len(words)))]
        assert vocab.tokenize(text, bos=True) == T.tokenize(text, True, *oracle_vocab), text


def test_empty_text(vocab, oracle_vocab):
    assert vocab.tokenize("", bos=True) == [1] == T.tokenize(b"", True, *oracle_vocab)
    assert vocab.tokenize("", bos=False) == [] == T.tokenize(b"", False, *oracle_vocab)


def test_pieces_and_scores(vocab, oracle_vocab):
    pieces, scores, _ = oracle_vocab
    for i in list(range(0, 300)) + [len(pieces) - 1]:
        assert vocab.piece(i) == pieces[i]
        assert vocab.score(i) == np.float32(scores[i])
    assert vocab.piece(3) == b"\x00" and vocab.piece(258) == b"\xff"   # byte tokens ignore the file's text
    with pytest.raises(IndexError):
        vocab.piece(len(pieces))


def test_hand_worked_merges(tmp_path):
    # ids: 259 " a" (-1), 260 "ab" (-2), 261 " ab" (-0.5), 262 "aa" (-1), 263 "b" (-3), 264 "b" again (-0.1)
    extra = [(b" a", -1.0), (b"ab", -2.0), (b" ab", -0.5), (b"aa", -1.0), (b"b", -3.0), (b"b", -0.1)]
    path = str(tmp_path / "vocab")
    write_vocab(path, base_entries() + extra)
    v = P.Vocabulary(path)
    ov = T.read_vocab(open(path, "rb").read())
    # "ab" -> " ab": pairs " a" (-1) and "ab" (-2); " a" merges first, then " a"+"b" = " ab" is known
    assert v.tokenize("ab", bos=False) == [261] == T.tokenize(b"ab", False, *ov)
    # " aaa": both "aa" pairs score -1, the left one merges; the second "a" is gone, the third stays a byte
    assert v.tokenize(" aaa", bos=False) == [259, 262] == T.tokenize(b" aaa", False, *ov)
    # "aaa" -> " aaa" the same way; "aab": " a" (-1) and "aa" (-1) tie -> leftmost " a" wins, then "ab"
    assert v.tokenize("aaa", bos=True) == [1, 259, 262]
    assert v.tokenize("aab", bos=False) == [259, 260] == T.tokenize(b"aab", False, *ov)
    # a repeated text resolves to its first id (263, not 264); single bytes below id 259 are never looked up
    assert v.tokenize("bb", bos=False) == [ord(" ") + 3, 263, 263] == T.tokenize(b"bb", False, *ov)
    v.close()


def test_malformed_vocab_files_are_refused(tmp_path):
    good = str(tmp_path / "good")
    write_vocab(good, base_entries() + [(b" a", -1.0)])
    data = open(good, "rb").read()
    P.Vocabulary(good).close()
    cases = {
        "empty": b"",
        "truncated table": data[:4 + 8 * 100],
        "no final NUL": data[:-1] + b"x",
        "offset past the end": data[:4 + 8 * 259] + struct.pack("<if", len(data) + 5, -1.0) + data[4 + 8 * 260:],
        "offset into the table": data[:4] + struct.pack("<if", 8, 0.0) + data[12:],
        "count too large": struct.pack("<i", 40000) + data[4:],
    }
    for name, blob in cases.items():
        path = str(tmp_path / "bad")
        open(path, "wb").write(blob)
        with pytest.raises(P.LcuError):
            P.Vocabulary(path)
    with pytest.raises(P.LcuError):
        P.Vocabulary(str(tmp_path / "missing"))
