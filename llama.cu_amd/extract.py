#!/usr/bin/env python3
"""Turns a LLaMA checkpoint into a model directory: the counterpart of the reference's extract.py.

    python extract.py weights <consolidated.pth> <model_dir>
    python extract.py params  <params.json>      <model_dir>/params  [--n-vocab 32000]
    python extract.py vocab   <tokenizer.model>  <model_dir>/vocab

File formats (extract.py:10-61 of the reference): every tensor of the state dict as raw little-endian
fp16 in `<key>__<d0>_<d1>...`; `params` = the 40-byte llama_params record (magic, fourcc, dim,
multiple_of, n_heads, n_layers, n_vocab, norm_eps, quantisation type 0 + block 0); `vocab` = int32
count, count x {int32 offset, float score}, then the NUL-terminated UTF-8 pieces with U+2581 written
as a space.  The checkpoint is read with torch.load(weights_only=True): nothing in it is executed.
"""
import argparse
import json
import os
import struct
import sys

LLAMA_CU_MAGIC = 0x000041524F525541   # "AURORA\0\0"
FOURCC_LLMA = 0x414D4C4C              # "LLMA"


def extract_weights(checkpoint, model_dir, log=print):
    import torch
    os.makedirs(model_dir, exist_ok=True)
    log("loading weights...")
    state = torch.load(checkpoint, map_location="cpu", weights_only=True)
    written = []
    for key, tensor in state.items():
        if not hasattr(tensor, "shape"):
            continue
        half = tensor.detach().to(dtype=torch.float16).contiguous()
        name = "%s__%s" % (key, "_".join(str(d) for d in half.shape))
        path = os.path.join(model_dir, name)
        log("writing %s..." % path)
        with open(path, "wb") as f:
            f.write(half.numpy().tobytes())
        written.append(name)
    return written


def pack_params(config, n_vocab=32000):
    return struct.pack("<QIiiiiifi", LLAMA_CU_MAGIC, FOURCC_LLMA, int(config["dim"]), int(config["multiple_of"]),
                       int(config["n_heads"]), int(config["n_layers"]), int(n_vocab), float(config["norm_eps"]), 0)


def extract_params(params_json, output_file, n_vocab=32000):
    with open(params_json) as f:
        config = json.load(f)
    os.makedirs(os.path.dirname(os.path.abspath(output_file)), exist_ok=True)
    with open(output_file, "wb") as f:
        f.write(pack_params(config, n_vocab))


def extract_vocab(tokenizer_model, output_file):
    from sentencepiece import SentencePieceProcessor
    sp = SentencePieceProcessor(model_file=tokenizer_model)
    n = sp.vocab_size()
    pieces = [sp.id_to_piece(i).replace("▁", " ").encode("utf-8") for i in range(n)]
    os.makedirs(os.path.dirname(os.path.abspath(output_file)), exist_ok=True)
    offset = 4 + 8 * n
    with open(output_file, "wb") as f:
        f.write(struct.pack("<i", n))
        for i, piece in enumerate(pieces):
            f.write(struct.pack("<if", offset, sp.get_score(i)))
            offset += len(piece) + 1
        for piece in pieces:
            f.write(piece + b"\0")
    return n


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)
    w = sub.add_parser("weights")
    w.add_argument("input_file")
    w.add_argument("output_dir")
    p = sub.add_parser("params")
    p.add_argument("input_file")
    p.add_argument("output_file")
    p.add_argument("--n-vocab", type=int, default=32000)
    v = sub.add_parser("vocab")
    v.add_argument("input_file")
    v.add_argument("output_file")
    a = ap.parse_args(argv)
    if a.command == "weights":
        extract_weights(a.input_file, a.output_dir)
    elif a.command == "params":
        extract_params(a.input_file, a.output_file, a.n_vocab)
    else:
        extract_vocab(a.input_file, a.output_file)
    return 0


if __name__ == "__main__":
    sys.exit(main())
