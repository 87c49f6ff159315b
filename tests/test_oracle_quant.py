"""Pins the oracle's int8 absmax quantiser (transform.cu:28-87) without the reference: a
hand-computed known-answer block, an exhaustive sweep against an independent numpy
float32/float16 restatement, and the invariants the algorithm fixes."""
import numpy as np

import oracle_lib as O


def np_quant_block(x16):
    """Independent numpy restatement for one block (IEEE float32 ops, half-away rounding)."""
    x = x16.astype(np.float32)
    absmax = np.max(np.abs(x)).astype(np.float32)
    scale16 = np.float16(absmax / np.float32(127.5))
    s = np.float32(scale16)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = np.float32(127.5) + x / s
    r = np.where(v >= 0, np.floor(v + np.float32(0.5)), np.ceil(v - np.float32(0.5)))
    # floor(v + 0.5) in float32 can round up for v just below a half; redo exactly in float64
    v64 = v.astype(np.float64)
    r = np.where(v64 >= 0, np.floor(v64 + 0.5), np.ceil(v64 - 0.5))
    return np.clip(r, 0, 255).astype(np.uint8), scale16


def test_known_answer_block():
    blk = np.zeros(128, dtype=np.float16)
    blk[:5] = [1.0, -1.0, 0.0, 0.5, -0.5]
    codes, scales = O.quantize_absmax_u8(blk.reshape(1, 128), 128)
    assert scales.view(np.uint16)[0, 0] == 0x2004  # fp16(1/127.5) = 0.007843017578125
    assert float(scales[0, 0]) == 0.007843017578125
    assert codes[0, :5].tolist() == [255, 0, 128, 191, 64]
    assert (codes[0, 5:] == 128).all()  # 127.5 rounds half away from zero
    deq = O.dequantize_absmax_u8(np.array([[0, 127, 128, 255] + [128] * 124], dtype=np.uint8), scales, 128)
    assert deq[0, :4].astype(np.float64).tolist() == [-1.0, -0.0039215087890625, 0.0039215087890625, 1.0]


def test_exhaustive_fp16_inputs_against_numpy():
    # every finite fp16 value as x, inside blocks whose absmax is set by a planted element
    allbits = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = allbits[np.isfinite(allbits)]
    for absmax in [np.float16(65504.0), np.float16(1.0), np.float16(0.0604), np.float16(3e-4), np.float16(6.1e-5)]:
        xs = finite[np.abs(finite) <= absmax]
        n = (len(xs) + 126) // 127
        blocks = np.zeros((n, 128), dtype=np.float16)
        blocks[:, 0] = absmax
        flat = np.zeros(n * 127, dtype=np.float16)
        flat[: len(xs)] = xs
        blocks[:, 1:] = flat.reshape(n, 127)
        codes, scales = O.quantize_absmax_u8(blocks, 128)
        for b in range(0, n, max(1, n // 64)):
            ec, es = np_quant_block(blocks[b])
            assert es.view(np.uint16) == scales[b, 0].view(np.uint16)
            assert (ec == codes[b]).all()
        # all blocks share absmax, so one vectorised check covers every input value
        s = np.float32(scales[0, 0])
        v = (np.float32(127.5) + blocks.astype(np.float32) / s).astype(np.float64)
        exp = np.clip(np.where(v >= 0, np.floor(v + 0.5), np.ceil(v - 0.5)), 0, 255).astype(np.uint8)
        assert (exp == codes).all()


def test_invariants_random():
    w = O.fill_normal_f16(64 * 1024, 3, 7, 0.02).reshape(64, 1024)
    codes, scales = O.quantize_absmax_u8(w, 128)
    wb = w.reshape(64, 8, 128).astype(np.float32)
    absmax = np.abs(wb).max(axis=2)
    assert (scales.view(np.uint16) == (absmax / np.float32(127.5)).astype(np.float16).view(np.uint16)).all()
    cb = codes.reshape(64, 8, 128)
    idx = np.abs(wb).argmax(axis=2)
    top = np.take_along_axis(cb, idx[..., None], axis=2)[..., 0]
    assert np.isin(top, [0, 255]).all()  # the absmax element lands on an end code
    deq = O.dequantize_absmax_u8(codes, scales, 128).astype(np.float32).reshape(64, 8, 128)
    s = scales.astype(np.float32)[..., None]
    assert (np.abs(deq - wb) <= s * 0.5 + np.abs(wb) * 2.0 ** -10 + 1e-7).all()
    # dequantise closed form: (q - 127.5) * scale is exact in fp32, one rounding to fp16
    exp = ((cb.astype(np.float32) - np.float32(127.5)) * s).astype(np.float16)
    assert (exp.view(np.uint16) == deq.astype(np.float16).view(np.uint16)).all()


def test_other_block_sizes():
    w = O.fill_normal_f16(16 * 512, 5, 9, 1.0).reshape(16, 512)
    for block in (32, 64, 256, 512):
        codes, scales = O.quantize_absmax_u8(w, block)
        assert scales.shape == (16, 512 // block)
        for r in (0, 15):
            for b in range(512 // block):
                ec, es = np_quant_block(w[r, b * block:(b + 1) * block])
                assert (ec == codes[r, b * block:(b + 1) * block]).all()
                assert es.view(np.uint16) == scales[r, b].view(np.uint16)


def test_zero_block_is_defined():
    codes, scales = O.quantize_absmax_u8(np.zeros((1, 128), dtype=np.float16), 128)
    assert scales[0, 0] == 0 and (codes == 0).all()


def test_fill_normal_statistics_and_determinism():
    a = O.fill_normal_f16(1 << 20, 0, 1, 0.02)
    b = O.fill_normal_f16(1 << 20, 0, 1, 0.02)
    assert (a.view(np.uint16) == b.view(np.uint16)).all()
    c = O.fill_normal_f16(1 << 20, 0, 2, 0.02)
    assert (a.view(np.uint16) != c.view(np.uint16)).mean() > 0.9
    x = a.astype(np.float64)
    assert abs(x.mean()) < 1e-4 and abs(x.std() - 0.02) < 2e-4
    # independent restatement of the recipe in Python integers
    M = (1 << 64) - 1

    def sm(z):
        z = (z + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)

    key = sm(0 ^ ((1 * 0xD1B54A32D192ED03) & M))
    scale = np.float32(0.02 / np.sqrt(8.0 * (65536.0 ** 2 - 1.0) / 12.0))
    for i in (0, 1, 12345, (1 << 20) - 1):
        h1 = sm((key + i) & M)
        h2 = sm(h1)
        s = sum((h >> sh) & 0xFFFF for h in (h1, h2) for sh in (0, 16, 32, 48)) - 262140
        assert np.float16(np.float32(s) * scale).view(np.uint16) == a[i].view(np.uint16)
