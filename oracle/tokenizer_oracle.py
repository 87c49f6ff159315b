"""TEST INFRASTRUCTURE ONLY: plain-Python restatement of the reference's vocabulary reader and
tokenizer (llama_cu.cu:1312-1437, llama_cu.h:316-358).  Only tests/ may import it.

Pinned by tests/test_tokenizer.py: against SentencePiece itself (a byte-fallback BPE model trained
in this container, committed as a vocab file in the reference's format together with
SentencePiece's own encodings of the test strings), and by hand-worked merges on a tiny vocabulary.
The reference ships no tokenizer model and no test vectors; parity with the LLaMA vocabulary
itself is unpinned (the file is not in the container).
"""
import heapq
import struct


def read_vocab(data):
    """llama_vocabulary::llama_vocabulary (llama_cu.cu:1318-1342): returns (pieces, scores, lookup).

    File: uint32 count; count x {uint32 offset, float score}; NUL-terminated piece texts at the
    offsets.  Ids 3..258 are the bytes 0..255 whatever the file says; only ids >= 259 can be
    found by text, and the first id wins for a repeated text."""
    (count,) = struct.unpack_from("<I", data, 0)
    pieces, scores, lookup = [], [], {}
    for i in range(count):
        offset, score = struct.unpack_from("<If", data, 4 + 8 * i)
        if 3 <= i < 259:
            text = bytes([i - 3])
        else:
            end = data.index(b"\0", offset)
            text = bytes(data[offset:end])
        pieces.append(text)
        scores.append(score)
        if i >= 259:
            lookup.setdefault(text, i)
    return pieces, scores, lookup


def _utf8_len(first):
    # llama_cu.cu:1312-1316: length from the high nibble of the first byte
    return (1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 3, 4)[first >> 4]


def tokenize(text, bos, pieces, scores, lookup):
    """llama_vocabulary::tokenize + llama_tokenizer::tokenize (llama_cu.cu:1344-1437).  text: bytes."""
    out = [1] if bos else []
    if not text:
        return out
    if text[0:1] != b" ":
        text = b" " + text                               # 1353-1358
    # one symbol per UTF-8 character, doubly linked by index (1366-1377)
    sym, pos = [], 0
    while pos < len(text):
        n = min(len(text) - pos, _utf8_len(text[pos]))
        sym.append([pos, n, len(sym) - 1, len(sym) + 1])  # start, length, prev, next
        pos += n
    sym[-1][3] = -1
    heap = []

    def try_add(left, right):                            # 1421-1437
        if left == -1 or right == -1:
            return
        joined = text[sym[left][0]:sym[left][0] + sym[left][1] + sym[right][1]]
        tid = lookup.get(joined)
        if tid is None:
            return
        # the reference's queue pops the highest score, the smaller left index on ties
        # (llama_cu.h:342-346); entries equal in both are the same merge, so their order is moot
        heapq.heappush(heap, (-scores[tid], left, right, len(joined)))

    for i in range(1, len(sym)):
        try_add(i - 1, i)
    while heap:                                          # 1382-1405
        _, left, right, size = heapq.heappop(heap)
        ls, rs = sym[left], sym[right]
        if ls[1] == 0 or rs[1] == 0 or ls[1] + rs[1] != size:
            continue
        ls[1] += rs[1]
        rs[1] = 0
        ls[3] = rs[3]
        if rs[3] >= 0:
            sym[rs[3]][2] = left
        try_add(ls[2], left)
        try_add(left, ls[3])
    i = 0
    while i != -1:                                       # 1406-1419
        start, n = sym[i][0], sym[i][1]
        piece = text[start:start + n]
        tid = lookup.get(piece)
        if tid is None:
            out.extend(b + 3 for b in piece)
        else:
            out.append(tid)
        i = sym[i][3]
    return out
