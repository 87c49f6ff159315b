"""The command line programs (llama.cu_amd/bin, built by build.py) and the model-directory loader,
on model directories written in the reference's format."""
import json
import os
import re
import struct
import subprocess

import numpy as np
import pytest

import model_dir as MD
import oracle_lib as O

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "..", "llama.cu_amd", "bin")
VOCAB = os.path.join(HERE, "golden", "spm_bpe_vocab.bin")
CFG = dict(dim=256, multiple_of=128, n_heads=2, n_layers=2, n_vocab=640)   # n_vocab = the fixture vocabulary
SEED, STD = 5, 0.05


@pytest.fixture(scope="module")
def gpu():
    import gpu_helpers as G
    G.setup()
    yield G
    G.release()


def run(tool, args, cwd, ok=True):
    exe = os.path.join(BIN, tool)
    assert os.path.exists(exe), "%s is missing: build it with `python llama.cu_amd/build.py`" % exe
    p = subprocess.run([exe] + [str(a) for a in args], cwd=str(cwd), capture_output=True, timeout=300)
    out, err = p.stdout.decode("utf-8", "replace"), p.stderr.decode("utf-8", "replace")
    if ok:
        assert p.returncode == 0, "%s %s failed (%d)\n%s\n%s" % (tool, args, p.returncode, out, err)
    return p.returncode, out, err


@pytest.fixture(scope="module")
def models(tmp_path_factory, gpu):
    root = tmp_path_factory.mktemp("work")
    tensors = MD.write_fp16_model(str(root / "models" / "tiny"), CFG, SEED, STD, vocab_file=VOCAB)
    rc, out, err = run("transform", ["quantize", "tiny", "tiny_q8", 128], root)
    return root, tensors, out


def test_transform_quantize_files_and_report(models):
    root, tensors, out = models
    qdir = root / "models" / "tiny_q8"
    reports = re.findall(r"quantizing (\S+) \((\d+) x (\d+)\)\n  rms/max/mean error: (\S+)/(\S+)/(\S+)", out)
    assert [r[0] for r in reports] == [m[0] for m in MD.matrices(CFG)]      # the reference's tensor order
    for (stem, _, rows, cols), rep in zip(MD.matrices(CFG), reports):
        w = tensors[stem]
        codes, scales = O.quantize_absmax_u8(w, 128)
        got_codes = np.fromfile(str(qdir / ("%s.weight__%d_%d" % (stem, rows, cols))), dtype=np.uint8)
        got_scales = np.fromfile(str(qdir / ("%s.scale__%d_%d" % (stem, rows, cols // 128))), dtype=np.uint16)
        assert (got_codes == codes.ravel()).all(), stem                      # bit-exact codes
        assert (got_scales == scales.view(np.uint16).ravel()).all(), stem    # bit-exact scales
        mse, mx, mean = O.error_stats(w, O.dequantize_absmax_u8(codes, scales, 128))
        assert (int(rep[1]), int(rep[2])) == (rows, cols)
        assert np.allclose([float(rep[3]), float(rep[4]), float(rep[5])], [np.sqrt(mse), mx, mean], rtol=1e-4, atol=2e-6)
    for stem in MD.vectors(CFG):
        name = "%s.weight__%d" % (stem, CFG["dim"])
        assert open(str(qdir / name), "rb").read() == open(str(root / "models" / "tiny" / name), "rb").read()
    want = MD.pack_params(CFG["dim"], CFG["multiple_of"], CFG["n_heads"], CFG["n_layers"], CFG["n_vocab"], 1e-6, 1, 128)
    assert open(str(qdir / "params"), "rb").read() == want
    assert open(str(qdir / "vocab"), "rb").read() == open(VOCAB, "rb").read()


def test_transform_histogram(models):
    root, tensors, _ = models
    rc, out, err = run("transform", ["histogram", "tiny_q8", "feed_forward.w2", 1], root)
    codes, _ = O.quantize_absmax_u8(tensors["layers.1.feed_forward.w2"], 128)
    want = np.bincount(codes.ravel(), minlength=256)
    lines = out.strip().split("\n")
    assert lines[0].split() == ["%X" % j for j in range(16)]
    got = []
    for i, line in enumerate(lines[1:17]):
        head, rest = line.split(":")
        assert head.strip() == "%X" % i
        got += [int(x) for x in rest.split()]
    assert got == want.tolist() and sum(got) == codes.size
    rc, out, err = run("transform", ["histogram", "tiny_q8", "output", -1], root)
    assert sum(int(x) for l in out.strip().split("\n")[1:17] for x in l.split(":")[1].split()) == 640 * 256


def test_transform_error_paths(models):
    root, _, _ = models
    rc, out, err = run("transform", ["quantize", "tiny_q8", "again"], root, ok=False)
    assert rc == 1 and "Input model is not fp16" in err
    rc, out, err = run("transform", ["histogram", "tiny"], root, ok=False)
    assert rc == 1 and "Input model is not uint8" in err
    rc, out, err = run("transform", ["histogram", "tiny_q8", "attention.wz"], root, ok=False)
    assert rc == 1 and "Unknown tensor name" in err
    rc, out, err = run("transform", ["histogram", "tiny_q8", "output", 0], root, ok=False)
    assert rc == 1 and "Invalid layer index" in err
    rc, out, err = run("transform", ["quantize", "nowhere", "x"], root, ok=False)
    assert rc == 1 and "Could not load params file" in err
    rc, out, err = run("transform", ["quantize", "tiny", "x", 100], root, ok=False)
    assert rc == 1 and "Unsupported block size" in err
    rc, out, err = run("transform", ["svd", "tiny"], root, ok=False)
    assert rc == 1


@pytest.mark.parametrize("q_type", [0, 1])
def test_loaded_model_equals_synthetic_model(models, gpu, q_type):
    """llama_model::load on the written directory against create_synthetic with the same seed:
    same tensors, and therefore the same logits, bit for bit."""
    G = gpu
    root, _, _ = models
    loaded = G.P.Model(path=str(root / "models" / ("tiny_q8" if q_type else "tiny")), context_len=256)
    synth = G.P.Model(**CFG, q_type=q_type, seed=SEED, weight_std=STD)
    assert (loaded.dim, loaded.n_vocab, loaded.q_type, loaded.qblock) == (256, 640, q_type, 128 if q_type else loaded.qblock)
    for stem, sid, rows, cols in MD.matrices(CFG):
        lw, ls = loaded.tensor(sid, rows, cols)
        sw, ss = synth.tensor(sid, rows, cols)
        assert lw.tobytes() == sw.tobytes(), stem
        if q_type:
            assert ls.tobytes() == ss.tobytes(), stem
    toks = np.random.default_rng(1).integers(3, CFG["n_vocab"], 40).astype(np.int16)
    lc = G.P.Context(loaded, context_len=256, temperature=0.8)
    sc = G.P.Context(synth, context_len=256, temperature=0.8)
    assert lc.next_token(toks) == sc.next_token(toks)
    assert lc.logits().tobytes() == sc.logits().tobytes()
    for o in (lc, sc, loaded, synth):
        o.close()


def test_model_load_failures(models, gpu, tmp_path):
    root, _, _ = models
    with pytest.raises(gpu.P.LcuError):
        gpu.P.Model(path=str(root / "models" / "missing"))
    # a directory with a tensor of the wrong size is refused, not read out of bounds
    broken = tmp_path / "broken"
    MD.write_fp16_model(str(broken), CFG, SEED, STD)
    with open(str(broken / "layers.1.attention.wo.weight__256_256"), "wb") as f:
        f.write(b"\0" * 100)
    with pytest.raises(gpu.P.LcuError):
        gpu.P.Model(path=str(broken))
    # bad magic in params
    bad = tmp_path / "badparams"
    MD.write_fp16_model(str(bad), CFG, SEED, STD)
    data = bytearray(open(str(bad / "params"), "rb").read())
    data[0] ^= 0xFF
    open(str(bad / "params"), "wb").write(bytes(data))
    with pytest.raises(gpu.P.LcuError):
        gpu.P.Model(path=str(bad))


def expected_generation(G, model_path, prompt, max_tokens, context_len, sample_seed=None):
    """The generation loop of main.cpp:69-100 driven from Python through the C handles."""
    vocab = G.P.Vocabulary(VOCAB)
    model = G.P.Model(path=model_path, context_len=context_len)
    ctx = G.P.Context(model, context_len=context_len, temperature=0.8)
    if sample_seed is not None:
        ctx.sample_with_seed(sample_seed)
    feed = vocab.tokenize(prompt, bos=True)
    history, text, n_prompt, generated = list(feed), b"", len(feed), 0
    while generated < max_tokens:
        if ctx.tokens_left() == 0:
            ctx.clear_tokens()
            feed = history[-(context_len // 2):]
        tok = ctx.next_token(np.array(feed, dtype=np.int16))
        if tok == 2:
            break
        text += vocab.piece(tok)
        feed = [tok]
        history.append(tok)
        generated += 1
    for o in (ctx, model, vocab):
        o.close()
    return text, n_prompt, generated


@pytest.mark.parametrize("name,max_tokens,context_len", [("tiny", 24, 2048), ("tiny_q8", 24, 2048), ("tiny", 60, 32)])
def test_generation_program(models, gpu, name, max_tokens, context_len):
    """llama_cu on the written model: same text as the same loop driven through the library (with a
    32-token context the run refills the context from the last 16 tokens several times), and the
    times.txt report."""
    root, _, _ = models
    prompt = "Building a website can be done in 10 easy steps:"
    rc, out, err = run("llama_cu", [4, name, prompt, max_tokens, context_len], root)
    text, n_prompt, generated = expected_generation(gpu, str(root / "models" / name), prompt, max_tokens, context_len)
    raw = subprocess.run([os.path.join(BIN, "llama_cu"), "4", name, prompt, str(max_tokens), str(context_len)],
                         cwd=str(root), capture_output=True, timeout=300).stdout
    marker = raw.index(b"Context memory:")
    body = raw[raw.index(b"\n", marker) + 1:]
    tail = ("\ntokens: %d time: " % generated).encode()
    assert body.startswith(text + tail), (body[:200], text[:200])
    assert "Dimension: 256" in out and "Vocab: 640" in out and "Layers: 2" in out
    times = open(str(root / "times.txt")).read().split()
    assert int(times[0]) == n_prompt and len(times) == 1 + generated
    assert all(float(t) > 0 for t in times[1:])


def test_generation_program_with_sample_seed(models, gpu):
    """The optional sample_seed argument: tokens drawn from the probabilities, reproducibly."""
    root, _, _ = models
    prompt = "Building a website"
    text, _, generated = expected_generation(gpu, str(root / "models" / "tiny"), prompt, 20, 64, sample_seed=77)
    greedy_text, _, _ = expected_generation(gpu, str(root / "models" / "tiny"), prompt, 20, 64)
    assert text != greedy_text
    raw = subprocess.run([os.path.join(BIN, "llama_cu"), "4", "tiny", prompt, "20", "64", "77"], cwd=str(root),
                         capture_output=True, timeout=300).stdout
    marker = raw.index(b"Context memory:")
    body = raw[raw.index(b"\n", marker) + 1:]
    assert body.startswith(text + ("\ntokens: %d time: " % generated).encode()), (body[:200], text[:200])


def test_generation_program_failures(models):
    root, _, _ = models
    rc, out, err = run("llama_cu", [4, "nowhere"], root, ok=False)
    assert rc == 1 and "Could not load params file" in err
    novocab = root / "models" / "novocab"
    MD.write_fp16_model(str(novocab), CFG, SEED, STD)
    rc, out, err = run("llama_cu", [4, "novocab"], root, ok=False)
    assert rc == 1 and "Could not load vocab file" in err
    rc, out, err = run("llama_cu", [4, "tiny", "x " * 100, 4, 16], root, ok=False)
    assert rc == 1 and "exceeds the context" in err
