"""Writes model directories in the reference's on-disk format (llama_cu.cu:929-984, extract.py:10-41)
from the seeded synthetic recipe, for the loader / transform / generation tests."""
import os
import shutil
import struct

import numpy as np

import oracle_lib as O

LLAMA_CU_MAGIC = 0x000041524F525541
FOURCC_LLMA = 0x414D4C4C
MATRIX_NAMES = ["attention.wq", "attention.wk", "attention.wv", "attention.wo", "feed_forward.w1", "feed_forward.w2",
                "feed_forward.w3"]


def ffn_dim(dim, multiple_of):
    # llama_cu.cu:765-767
    return multiple_of * ((2 * 4 * dim // 3 + multiple_of - 1) // multiple_of)


def pack_params(dim, multiple_of, n_heads, n_layers, n_vocab, norm_eps=1e-6, q_type=0, qblock=0):
    # llama_cu.h:280-291: 40 bytes, little endian, no padding
    return struct.pack("<QIIIIIIfBBH", LLAMA_CU_MAGIC, FOURCC_LLMA, dim, multiple_of, n_heads, n_layers, n_vocab,
                       norm_eps, q_type, 0, qblock)


def matrices(cfg):
    """(file stem, synthetic stream id, rows, cols) of every weight matrix"""
    dim, ffn, vocab = cfg["dim"], ffn_dim(cfg["dim"], cfg["multiple_of"]), cfg["n_vocab"]
    out = [("tok_embeddings", 1, vocab, dim), ("output", 2, vocab, dim)]
    shapes = [(dim, dim)] * 4 + [(ffn, dim), (dim, ffn), (ffn, dim)]
    for l in range(cfg["n_layers"]):
        for j, name in enumerate(MATRIX_NAMES):
            out.append(("layers.%d.%s" % (l, name), 16 + 16 * l + j, shapes[j][0], shapes[j][1]))
    return out


def vectors(cfg):
    return ["norm"] + ["layers.%d.%s" % (l, n) for l in range(cfg["n_layers"]) for n in ("attention_norm", "ffn_norm")]


def write_fp16_model(path, cfg, seed, weight_std, vocab_file=None, norm_eps=1e-6):
    """fp16 model directory whose tensors equal llama_model::create_synthetic(cfg, seed, weight_std).
    Returns {file stem: fp16 array}."""
    os.makedirs(path, exist_ok=True)
    tensors = {}
    for stem, sid, rows, cols in matrices(cfg):
        w = O.fill_normal_f16(rows * cols, seed, sid, weight_std).reshape(rows, cols)
        w.tofile(os.path.join(path, "%s.weight__%d_%d" % (stem, rows, cols)))
        tensors[stem] = w
    for stem in vectors(cfg):
        np.ones(cfg["dim"], dtype=np.float16).tofile(os.path.join(path, "%s.weight__%d" % (stem, cfg["dim"])))
    with open(os.path.join(path, "params"), "wb") as f:
        f.write(pack_params(cfg["dim"], cfg["multiple_of"], cfg["n_heads"], cfg["n_layers"], cfg["n_vocab"], norm_eps))
    if vocab_file:
        shutil.copy(vocab_file, os.path.join(path, "vocab"))
    return tensors
