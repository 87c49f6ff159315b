"""The checkpoint extractor (llama.cu_amd/extract.py) on a small fabricated checkpoint: file names,
fp16 payloads, the params record and the vocabulary file."""
import importlib.util
import json
import os
import struct

import numpy as np
import pytest

import model_dir as MD

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
spec = importlib.util.spec_from_file_location("lcu_extract", os.path.join(HERE, "..", "llama.cu_amd", "extract.py"))
X = importlib.util.module_from_spec(spec)
spec.loader.exec_module(X)


def test_weights_become_raw_fp16_files(tmp_path):
    torch = pytest.importorskip("torch")
    g = torch.Generator().manual_seed(0)
    state = {
        "tok_embeddings.weight": torch.randn(40, 16, generator=g),
        "norm.weight": torch.ones(16, dtype=torch.bfloat16),
        "layers.0.attention.wq.weight": torch.randn(16, 16, generator=g).to(torch.float16),
        "layers.0.feed_forward.w1.weight": torch.randn(48, 16, generator=g, dtype=torch.float64),
        "rope.freqs": torch.arange(8, dtype=torch.float32),
    }
    ckpt = str(tmp_path / "consolidated.00.pth")
    torch.save(state, ckpt)
    out = str(tmp_path / "models" / "fake")
    names = X.extract_weights(ckpt, out, log=lambda *_: None)
    assert sorted(names) == sorted(os.listdir(out))
    assert "tok_embeddings.weight__40_16" in names and "norm.weight__16" in names and "rope.freqs__8" in names
    for key, t in state.items():
        name = "%s__%s" % (key, "_".join(str(d) for d in t.shape))
        got = np.fromfile(os.path.join(out, name), dtype=np.float16).reshape(tuple(t.shape))
        assert (got.view(np.uint16) == t.to(torch.float16).numpy().view(np.uint16)).all(), key


def test_params_record(tmp_path):
    cfg = {"dim": 4096, "multiple_of": 256, "n_heads": 32, "n_layers": 32, "norm_eps": 1e-06, "vocab_size": -1}
    src = str(tmp_path / "params.json")
    json.dump(cfg, open(src, "w"))
    dst = str(tmp_path / "m" / "params")
    X.extract_params(src, dst)
    data = open(dst, "rb").read()
    assert len(data) == 40
    assert data == MD.pack_params(4096, 256, 32, 32, 32000, 1e-6, 0, 0)    # the record the loader tests write
    magic, fourcc = struct.unpack_from("<QI", data)
    assert magic == 0x000041524F525541 and fourcc == 0x414D4C4C
    X.main(["params", src, dst, "--n-vocab", "640"])
    assert struct.unpack_from("<i", open(dst, "rb").read(), 28)[0] == 640


def test_vocab_file_from_a_sentencepiece_model(tmp_path):
    pytest.importorskip("sentencepiece")
    dst = str(tmp_path / "vocab")
    n = X.extract_vocab(os.path.join(GOLDEN, "spm_bpe.model"), dst)
    assert n == 640
    # byte for byte the committed vocabulary fixture, which the tokenizer tests read through the library
    assert open(dst, "rb").read() == open(os.path.join(GOLDEN, "spm_bpe_vocab.bin"), "rb").read()
