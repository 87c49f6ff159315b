"""Pins the oracle's restatement of the reference kernels (llama_cu.cu:30-540) by what the
mathematics fixes: float64 brute force written independently in numpy, exact special cases,
and invariants.  Each check is chosen so that a dropped term, a wrong index or a transposed
operand fails it."""
from pathlib import Path

import numpy as np
import pytest

import oracle_lib as O

GOLDEN = Path(__file__).parent / "golden"
RNG = np.random.default_rng(1234)


def rel_err(a, ref):
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return np.max(np.abs(a - ref)) / max(np.max(np.abs(ref)), 1e-30)


def f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


# ------------------------------------------------------------------ matmul
@pytest.mark.parametrize("flavour", [0, 1, 2])
@pytest.mark.parametrize("M,K,N", [(1, 256, 64), (5, 272, 33), (16, 1024, 128), (3, 40, 7)])
def test_matmul_vs_float64(flavour, M, K, N):
    x = f16(RNG.normal(0, 1, (M, K)))
    w = f16(RNG.normal(0, 0.02, (N, K)))
    out = O.matmul_nt(x, w, flavour=flavour)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    # fp32 accumulation + one fp16 rounding
    assert np.max(np.abs(out.astype(np.float64) - ref)) <= np.max(np.abs(ref)) * 2.0 ** -10


@pytest.mark.parametrize("flavour", [0, 1, 2])
def test_matmul_exact_cases(flavour):
    K = 128
    x = f16(RNG.normal(0, 1, (4, K)))
    eye = np.eye(K, dtype=np.float16)
    assert (O.matmul_nt(x, eye, flavour=flavour).view(np.uint16) == x.view(np.uint16)).all()
    w = f16(RNG.normal(0, 0.02, (48, K)))
    onehot = np.zeros((1, K), dtype=np.float16)
    onehot[0, 37] = 1
    assert (O.matmul_nt(onehot, w, flavour=flavour)[0].view(np.uint16) == w[:, 37].view(np.uint16)).all()
    # asymmetric operand: out[m, n] pairs lhs row m with rhs row n (a transposed operand fails)
    w2 = np.zeros((3, K), dtype=np.float16)
    w2[2, 5] = 2
    x2 = np.zeros((2, K), dtype=np.float16)
    x2[1, 5] = 3
    out = O.matmul_nt(x2, w2, flavour=flavour)
    assert out[1, 2] == 6 and np.count_nonzero(out) == 1


@pytest.mark.parametrize("flavour", [0, 1, 2])
def test_matmul_beta_residual(flavour):
    x = f16(RNG.normal(0, 1, (3, 256)))
    w = f16(RNG.normal(0, 0.02, (20, 256)))
    old = f16(RNG.normal(0, 1, (3, 20)))
    out = O.matmul_nt(x, w, beta=1.0, out=old, flavour=flavour)
    ref = x.astype(np.float64) @ w.astype(np.float64).T + old.astype(np.float64)
    assert np.max(np.abs(out.astype(np.float64) - ref)) <= np.max(np.abs(ref)) * 2.0 ** -10
    # beta = 0 ignores whatever the output held
    junk = np.full((3, 20), np.inf, dtype=np.float16)
    assert np.isfinite(O.matmul_nt(x, w, beta=0.0, out=junk, flavour=flavour)).all()


@pytest.mark.parametrize("flavour", [0, 1, 2])
def test_matmul_u8_vs_float64_and_dequant_route(flavour):
    K, N, M, block = 512, 40, 3, 128
    w = f16(RNG.normal(0, 0.02, (N, K)))
    x = f16(RNG.normal(0, 1, (M, K)))
    codes, scales = O.quantize_absmax_u8(w, block)
    out = O.matmul_nt_u8(x, codes, scales, block, flavour=flavour)
    wd64 = (codes.astype(np.float64) - 127.5) * np.repeat(scales.astype(np.float64), block, axis=1)
    ref = x.astype(np.float64) @ wd64.T
    assert np.max(np.abs(out.astype(np.float64) - ref)) <= np.max(np.abs(ref)) * 2.0 ** -9
    if flavour == 1:
        # the tensor-core route is exactly "dequantise to fp16, then the fp16 matmul" (llama_cu.cu:331-342)
        wd = O.dequantize_absmax_u8(codes, scales, block)
        assert (O.matmul_nt(x, wd, flavour=1).view(np.uint16) == out.view(np.uint16)).all()


def test_matmul_row_independence():
    x = f16(RNG.normal(0, 1, (9, 256)))
    w = f16(RNG.normal(0, 0.02, (31, 256)))
    full = O.matmul_nt(x, w)
    for r in (0, 4, 8):
        assert (O.matmul_nt(x[r:r + 1], w).view(np.uint16) == full[r:r + 1].view(np.uint16)).all()


# ------------------------------------------------------------------ flavour 2 (one row in the order of the HIP GEMV kernels)
def fused_sum_numpy(a, b, c, step):
    with np.errstate(all="ignore"):
        return _fused_sum_numpy(a, b, c, step)


def _fused_sum_numpy(a, b, c, step):
    """What gfx950 does with fp16 products and an fp32 accumulator (v_dot2_f32_f16: step = 2 = K; the
    matrix cores: steps of 8 over ascending k), restated on its own in float64 from the measured
    samples under tests/golden/.  a, b of shape (n, K) hold halves, c fp32 values.  A half is
    m * 2^(e - 10) with e >= -14.  Per step: e = the largest e_a + e_b of the non-zero products;
    every product is cut towards zero to a multiple of 2^(e - 24) and c down to one; their exact sum
    keeps 32 significant bits (cut down) and is rounded to fp32, to nearest even."""
    a, b = a.astype(np.float64), b.astype(np.float64)
    acc = c.astype(np.float64)

    def expo(v, floor=None):
        e = np.frexp(np.abs(v))[1] - 1
        if floor is not None:
            e = np.maximum(e, floor)
        return np.where(v == 0, -10000, e)

    for k0 in range(0, a.shape[1], step):  # (steps without a non-zero product compute with 2^-10024 = 0 and are discarded)
        p = a[:, k0:k0 + step] * b[:, k0:k0 + step]
        e = np.where(p == 0, -10000, expo(a[:, k0:k0 + step], -14) + expo(b[:, k0:k0 + step], -14)).max(1)
        q = np.ldexp(1.0, e - 24)
        pp = (np.trunc(p / q[:, None]) * q[:, None]).sum(1)
        # with c far above the products pp + c would not fit float64; pp cut down to 2^(ec - 44) first
        # gives the same result (c is a multiple of it and the final cut is coarser)
        g = np.maximum(q, np.ldexp(1.0, expo(acc) - 44))
        S = np.floor(pp / g) * g + np.floor(acc / q) * q
        qr = np.ldexp(1.0, np.where(S == 0, 0, expo(S)) - 31)
        r = (np.floor(S / qr) * qr).astype(np.float32)
        acc = np.where(e <= -10000, acc.astype(np.float32), r).astype(np.float64)
    return acc.astype(np.float32)


def dot2_numpy(a, b, c):
    return fused_sum_numpy(a, b, c, 2)


def gemv_order_numpy(x, w, u8):
    """Independent restatement of dot_gemv_order.  fp16 weights: products of two halves are exact in
    fp32, so every fused multiply-add is a plain fp32 addition of an exact product.  uint8 weights:
    pairs of products through dot2_numpy."""
    K = x.size
    vec, U = (16, 1) if u8 else (8, 2)
    chunk = vec * 64
    acc = np.zeros((4, 64, 2), dtype=np.float32)
    prod = (x.astype(np.float32) * w.astype(np.float32)).astype(np.float32)
    lanes = np.arange(64)
    for c in range((K + chunk - 1) // chunk):
        wave = (c // U) % 4
        kk = c * chunk + lanes * vec
        ok = kk < K
        if u8:
            for e in range(0, vec, 2):
                which = (e % 4) // 2
                idx = np.where(ok, kk + e, 0)
                got = dot2_numpy(np.stack([w[idx], w[idx + 1]], 1), np.stack([x[idx], x[idx + 1]], 1), acc[wave, :, which])
                acc[wave, :, which] = np.where(ok, got, acc[wave, :, which])
            continue
        for e in range(vec):
            idx = np.where(ok, kk + e, 0)
            acc[wave, :, e % 2] = np.where(ok, (acc[wave, :, e % 2] + prod[idx]).astype(np.float32), acc[wave, :, e % 2])
    total = np.float32(0)
    for wave in range(4):
        v = (acc[wave, :, 0] + acc[wave, :, 1]).astype(np.float32)
        step = 1
        while step < 64:
            v[::2 * step] = (v[::2 * step] + v[step::2 * step]).astype(np.float32)
            step *= 2
        total = np.float32(total + v[0])
    return total


def test_dot2_against_the_gpu_samples():
    """The oracle's v_dot2_f32_f16 and the restatement above against what gfx950 returned
    (tests/golden/dot2_probe.hip made the samples, make_dot2_fixture.py chose them)."""
    z = np.load(GOLDEN / "dot2_gfx950.npz")
    a, b, c, want = z["a"], z["b"], z["c"].view(np.float32), z["out"]
    assert a.shape[0] > 10000
    got = O.dot2_f32_f16(a, b, c)
    assert (got.view(np.uint32) == want).all()
    mine = dot2_numpy(a.view(np.float16), b.view(np.float16), c)
    assert (mine.view(np.uint32) == want).all()
    # two fused multiply-adds would not do: the fixture tells them apart
    chain = np.float32(np.float32(a.view(np.float16)[:, 0].astype(np.float64) * b.view(np.float16)[:, 0] + c)
                       + a.view(np.float16)[:, 1].astype(np.float64) * b.view(np.float16)[:, 1])
    assert (chain.view(np.uint32) != want).sum() > 1000


def test_dot2_closed_forms():
    """What needs no measurement: exact sums come back exact, and c alone passes through."""
    h = lambda *v: np.array([v], dtype=np.float16).view(np.uint16)
    one = lambda a, b, c: float(O.dot2_f32_f16(h(*a), h(*b), np.array([c], dtype=np.float32))[0])
    assert one((1.5, 2.0), (2.0, 0.25), 1.0) == 4.5
    assert one((0.0, 0.0), (3.0, 4.0), 0.3) == float(np.float32(0.3))
    assert one((3.0, 0.0), (5.0, 1.0), 0.0) == 15.0
    assert one((-3.0, 2.0), (5.0, 7.5), 0.0) == 0.0
    assert one((-3.0, 2.0), (5.0, 7.0), 1.0) == 0.0                            # the three cancel exactly
    assert one((2.0 ** -20, 0.0), (2.0 ** -4, 0.0), 0.0) == 2.0 ** -24          # a subnormal half, exact
    assert one((1.0, 0.0), (1.0, 0.0), 2.0 ** 24) == 2.0 ** 24                  # tie to even
    assert one((1.0, 1.0), (1.0, 1.0), 2.0 ** 24) == 2.0 ** 24 + 2.0            # both products count before rounding
    assert one((1.0, 0.0), (2.0 ** -14, 0.0), 2.0 ** 80) == 2.0 ** 80           # c far above the products


def test_mfma_against_the_gpu_samples():
    """The oracle's matrix-core step and the restatement above against what gfx950 returned for
    v_mfma_f32_32x32x16_f16 (K = 16: two steps of eight; among them instructions out of K = 4096
    chains) and v_mfma_f32_16x16x32_f16 (K = 32: four); tests/golden/mfma_probe.hip made the
    samples, make_mfma_fixture.py chose them."""
    z = np.load(GOLDEN / "mfma_gfx950.npz")
    for K in (16, 32):
        a, b, c, want = z[f"a{K}"], z[f"b{K}"], z[f"c{K}"].view(np.float32), z[f"out{K}"]
        assert a.shape[0] > 3000 and a.shape[1] == K
        assert (O.mfma_f32_f16(a, b, c).view(np.uint32) == want).all()
        assert (fused_sum_numpy(a.view(np.float16), b.view(np.float16), c, 8).view(np.uint32) == want).all()
        # neither one rounding of the exact sum nor all K products in one step would do
        exact = (a.view(np.float16).astype(np.float64) * b.view(np.float16).astype(np.float64)).sum(1) + c
        assert (exact.astype(np.float32).view(np.uint32) != want).sum() > 300
        assert (fused_sum_numpy(a.view(np.float16), b.view(np.float16), c, K).view(np.uint32) != want).sum() > 200


def test_mfma_closed_forms():
    rng = np.random.default_rng(5)
    # small integers: every sum is exact whatever the order
    a = rng.integers(-8, 9, (64, 32)).astype(np.float16)
    b = rng.integers(-8, 9, (64, 32)).astype(np.float16)
    c = rng.integers(-100, 101, 64).astype(np.float32)
    want = (a.astype(np.float64) * b.astype(np.float64)).sum(1) + c
    assert (O.mfma_f32_f16(a.view(np.uint16), b.view(np.uint16), c) == want).all()
    # all products zero: c untouched, also a c that fp16 could not hold
    z = np.zeros((4, 16), dtype=np.float16)
    c = np.array([1e-30, -3.0e38, 0.1, 0.0], dtype=np.float32)
    assert (O.mfma_f32_f16(z.view(np.uint16), b[:4, :16].view(np.uint16), c).view(np.uint32) == c.view(np.uint32)).all()
    # a step whose products cancel c exactly gives 0, and the next step starts from it
    a = np.zeros((1, 16), dtype=np.float16)
    b = np.ones((1, 16), dtype=np.float16)
    a[0, 0], a[0, 1], a[0, 8] = 3, -1, 0.5
    assert O.mfma_f32_f16(a.view(np.uint16), b.view(np.uint16), np.array([-2.0], dtype=np.float32))[0] == 0.5


# (M, K, N, uint8, matrices per launch) -> (wavefront groups per K stage, K splits): the dispatcher of
# csrc/gemm.hip, restated for the oracle's kernel-order flavour
@pytest.mark.parametrize("shape,plan", [((512, 4096, 4096, False, 1), (2, 1)), ((512, 4096, 11008, False, 1), (1, 1)),
                                        ((512, 4096, 4096, False, 3), (1, 1)), ((512, 4096, 11008, False, 2), (1, 1)),
                                        ((32, 11008, 4096, True, 1), (1, 8)), ((2, 4096, 4096, False, 1), (1, 8)),
                                        ((8, 4096, 4096, False, 3), (1, 3)), ((130, 200, 70, False, 1), (2, 1)),
                                        ((512, 6656, 6656, True, 3), (1, 1)), ((64, 4096, 11008, False, 1), (1, 3)),
                                        ((512, 11008, 4096, False, 1), (1, 4)), ((512, 17920, 6656, True, 1), (1, 2))])
def test_gemm_plan(shape, plan):
    M, K, N, u8, n_mats = shape
    assert O.gemm_plan(M, K, N, u8, 128, n_mats) == plan


def gemm_order_numpy(x, w, ks, splits):
    """Independent restatement of the kernel-order matrix product: chains of steps of eight over
    ascending k from 0, K cut into chains by the plan, the chains added in order."""
    M, K = x.shape
    N = w.shape[0]
    if ks == 2:
        chains = [[k for k in range(0, K, 8) if (k // 64) % 2 == g] for g in range(2)]
    else:
        stages = K // 64
        chains = [list(range((s * stages // splits) * 64, ((s + 1) * stages // splits) * 64, 8)) for s in range(splits)] \
            if splits > 1 else [list(range(0, K, 8))]
    a = np.repeat(x, N, axis=0)          # row m * N + n: x[m]
    b = np.tile(w, (M, 1))               # and w[n]
    total = None
    for chain in chains:
        cols = np.concatenate([np.arange(k, k + 8) for k in chain]) if chain else np.zeros(0, dtype=int)
        acc = fused_sum_numpy(a[:, cols], b[:, cols], np.zeros(M * N, dtype=np.float32), 8) if len(cols) else \
            np.zeros(M * N, dtype=np.float32)
        total = acc if total is None else (total + acc).astype(np.float32)
    return total.reshape(M, N)


@pytest.mark.parametrize("M,K,N", [(7, 64, 24), (33, 200, 10), (5, 1024, 520), (40, 384, 12), (130, 256, 9)])
def test_kernel_order_product_fp16(M, K, N):
    x = f16(RNG.normal(0, 1, (M, K)))
    w = f16(RNG.normal(0, 0.02, (N, K)))
    ks, splits = O.gemm_plan(M, K, N)
    out = O.matmul_nt(x, w, flavour=2)
    want = gemm_order_numpy(x, w, ks, splits).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all(), (ks, splits)
    ref64 = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.max(np.abs(out.astype(np.float64) - ref64)) <= np.max(np.abs(ref64)) * 2.0 ** -10
    old = f16(RNG.normal(0, 1, (M, N)))
    out = O.matmul_nt(x, w, beta=1.0, out=old, flavour=2)
    want = (gemm_order_numpy(x, w, ks, splits) + old.astype(np.float32)).astype(np.float32).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all()
    # identity weights give x back, a one-hot row picks a column of w
    assert (O.matmul_nt(x[:, :64], np.eye(64, dtype=np.float16), flavour=2).view(np.uint16) == x[:, :64].view(np.uint16)).all()
    onehot = np.zeros((2, K), dtype=np.float16)
    onehot[1, K // 3] = 1
    assert (O.matmul_nt(onehot, w, flavour=2)[1].view(np.uint16) == w[:, K // 3].view(np.uint16)).all()


@pytest.mark.parametrize("M,K,N,n_mats", [(9, 256, 24, 1), (33, 1024, 300, 2), (5, 4096, 260, 3)])
def test_kernel_order_product_u8(M, K, N, n_mats):
    x = f16(RNG.normal(0, 1, (M, K)))
    w = f16(RNG.normal(0, 0.02, (N, K)))
    codes, scales = O.quantize_absmax_u8(w, 128)
    wd = O.dequantize_absmax_u8(codes, scales, 128)
    ks, splits = O.gemm_plan(M, K, N, True, 128, n_mats)
    out = O.matmul_nt_kernel_order(x, codes=codes, scales=scales, block=128, n_mats=n_mats)
    want = gemm_order_numpy(x, wd, ks, splits).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all(), (ks, splits)
    if n_mats == 1:
        assert (O.matmul_nt_u8(x, codes, scales, 128, flavour=2).view(np.uint16) == out.view(np.uint16)).all()


@pytest.mark.parametrize("K", [8, 512, 1032, 4096, 11008])
def test_single_row_kernel_order_fp16(K):
    x = f16(RNG.normal(0, 1, (1, K)))
    w = f16(RNG.normal(0, 0.02, (5, K)))
    out = O.matmul_nt(x, w, flavour=2)
    ref64 = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.max(np.abs(out.astype(np.float64) - ref64)) <= np.max(np.abs(ref64)) * 2.0 ** -10
    want = np.array([[gemv_order_numpy(x[0], w[n], False) for n in range(5)]], dtype=np.float32).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all()
    # residual: one rounding of the fp32 sum
    old = f16(RNG.normal(0, 1, (1, 5)))
    out = O.matmul_nt(x, w, beta=1.0, out=old, flavour=2)
    want = np.array([[np.float32(gemv_order_numpy(x[0], w[n], False) + np.float32(old[0, n])) for n in range(5)]],
                    dtype=np.float32).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all()
    # exact cases: a one-hot row picks a column of w
    onehot = np.zeros((1, K), dtype=np.float16)
    onehot[0, K // 3] = 1
    assert (O.matmul_nt(onehot, w, flavour=2)[0].view(np.uint16) == w[:, K // 3].view(np.uint16)).all()


@pytest.mark.parametrize("K", [128, 1024, 6656])
def test_single_row_kernel_order_u8(K):
    block = 128
    w = f16(RNG.normal(0, 0.02, (4, K)))
    x = f16(RNG.normal(0, 1, (1, K)))
    codes, scales = O.quantize_absmax_u8(w, block)
    wd = O.dequantize_absmax_u8(codes, scales, block)
    out = O.matmul_nt_u8(x, codes, scales, block, flavour=2)
    want = np.array([[gemv_order_numpy(x[0], wd[n], True) for n in range(4)]], dtype=np.float32).astype(np.float16)
    assert (out.view(np.uint16) == want.view(np.uint16)).all()
    ref64 = x.astype(np.float64) @ wd.astype(np.float64).T
    assert np.max(np.abs(out.astype(np.float64) - ref64)) <= np.max(np.abs(ref64)) * 2.0 ** -10


def test_exp_ieee_against_float64():
    x = np.concatenate([np.linspace(-90, 89, 200001), RNG.normal(0, 3, 100000), RNG.uniform(-20, 0, 100000),
                        [0.0, -0.0, 1.0, -1.0, 88.7, -87.3]]).astype(np.float32)
    got = O.exp_f32(x)
    ref = np.exp(x.astype(np.float64))
    normal = (ref >= 1.18e-38) & (ref < 3.4e38)
    ulp = np.spacing(ref[normal].astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got[normal].astype(np.float64) - ref[normal]) / ulp) <= 1.05  # CUDA documents 2 ulp for expf
    assert got[x == 0].tolist() == [1.0] * int((x == 0).sum())
    special = O.exp_f32(np.array([-np.inf, -200.0, 89.0, np.inf, np.nan], dtype=np.float32))
    assert special[0] == 0 and special[1] == 0 and np.isposinf(special[2]) and np.isposinf(special[3]) and np.isnan(special[4])
    # monotone on a dense grid (a softmax must not reorder its inputs)
    grid = np.linspace(-30, 10, 400001).astype(np.float32)
    assert (np.diff(O.exp_f32(grid)) >= 0).all()


@pytest.mark.parametrize("T", [1, 7, 64, 577, 1500])
def test_attention_decode_kernel_order(T):
    n_heads, dim = 3, 384
    q = f16(RNG.normal(0, 1, (1, dim)))
    k = f16(RNG.normal(0, 1, (T, dim)))
    v = f16(RNG.normal(0, 1, (T, dim)))
    got = O.attention_decode_kernel_order(q, k, v, n_heads)
    # same arithmetic as the reference-ordered chain: scores may differ by the last fp16 bit, so the
    # output follows it to fp16 rounding accuracy, and float64 attention within the usual bound
    ref = O.attention(q, k, v, n_heads, T - 1)
    assert np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64))) <= 2.0 ** -8 * np.max(np.abs(ref.astype(np.float64)))
    q64, k64, v64 = (a.astype(np.float64) for a in (q, k, v))
    for h in range(n_heads):
        sl = slice(h * 128, (h + 1) * 128)
        sc = k64[:, sl] @ q64[0, sl] / np.sqrt(128.0)
        p = np.exp(sc - sc.max())
        p /= p.sum()
        o = p @ v64[:, sl]
        assert np.max(np.abs(got[0, sl].astype(np.float64) - o)) <= 4e-3 * max(np.max(np.abs(o)), 0.05)
    if T == 1:
        assert (got.view(np.uint16) == v[:1].view(np.uint16)).all()  # a single row has probability 1


def attention_prefill_numpy(q, k, v, n_heads, start):
    """Independent restatement of attention_prefill_kernel_order with fused_sum_numpy and exp_f32."""
    n, dim = q.shape
    T = k.shape[0]
    BR = 16 if ((n + 31) // 32) * n_heads < 1024 and T <= 1024 else 32
    out = np.zeros((n, dim), dtype=np.float16)
    for h in range(n_heads):
        sl = slice(h * 128, (h + 1) * 128)
        for r in range(n):
            last = min(r // BR * BR + BR, n) - 1
            Tc = (min(T, last + start + 1) + 63) // 64 * 64
            vis = min(T, r + start + 1)
            acc = fused_sum_numpy(np.repeat(q[r:r + 1, sl], vis, 0), k[:vis, sl], np.zeros(vis, dtype=np.float32), 8)
            sc = np.full(Tc, -np.inf, dtype=np.float16)
            sc[:vis] = (acc / np.sqrt(np.float32(128.0))).astype(np.float16)
            x = sc.astype(np.float32)
            m = x.max()
            e = O.exp_f32(x - m)
            pair = (e[0::2] + e[1::2]).astype(np.float32)
            lanes = np.zeros(64, dtype=np.float32)
            for i in range(Tc // 2):  # lane i % 64 adds its pairs in ascending order
                lanes[i % 64] = np.float32(lanes[i % 64] + pair[i])
            step = 1
            while step < 64:
                lanes[::2 * step] = (lanes[::2 * step] + lanes[step::2 * step]).astype(np.float32)
                step *= 2
            p = (e / lanes[0]).astype(np.float32).astype(np.float16)
            vv = np.zeros((Tc, 128), dtype=np.float16)
            vv[:T] = v[:Tc, sl][:T]
            o = fused_sum_numpy(np.repeat(p[None, :], 128, 0), np.ascontiguousarray(vv.T), np.zeros(128, dtype=np.float32), 8)
            out[r, sl] = o.astype(np.float16)
    return out


@pytest.mark.parametrize("n,T", [(5, 5), (3, 130), (40, 70), (17, 17)])
def test_attention_prefill_kernel_order(n, T):
    n_heads, dim = 2, 256
    start = T - n
    q = f16(RNG.normal(0, 1, (n, dim)))
    k = f16(RNG.normal(0, 1, (T, dim)))
    v = f16(RNG.normal(0, 1, (T, dim)))
    got = O.attention_prefill_kernel_order(q, k, v, n_heads, start)
    assert (got.view(np.uint16) == attention_prefill_numpy(q, k, v, n_heads, start).view(np.uint16)).all()
    ref = O.attention(q, k, v, n_heads, start)
    assert np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64))) <= 2.0 ** -8 * np.max(np.abs(ref.astype(np.float64)))
    if start == 0:
        assert (got[0].view(np.uint16) == v[0].view(np.uint16)).all()  # causal row 0 sees only itself


def test_context_flavour_2_is_its_operators():
    """A flavour-2 context is the kernel-order operators chained: a prompt's hidden state equals what
    the exported pieces give on one layer (so the tests of the pieces carry over to the model)."""
    cfg = dict(dim=256, multiple_of=128, n_heads=2, n_layers=1, n_vocab=320)
    om = O.Model(**cfg, seed=2, weight_std=0.05)
    oc = O.Context(om, context_len=16, temperature=0.8, flavour=2)
    toks = np.array([3, 100, 7, 250, 9], dtype=np.int16)
    _, hid, _, _ = oc.next_token(toks, want=True)
    ffn = om.ffn
    w = {kind: om.tensor(16 + kind, *((ffn, 256) if kind in (4, 6) else ((256, ffn) if kind == 5 else (256, 256))))[0]
         for kind in range(7)}
    x = om.tensor(1, 320, 256)[0][toks]
    an = fn = np.ones(256, dtype=np.float16)  # synthetic models keep their norm weights at one
    nx = O.rms_norm(x, an, 1e-6)
    xq = O.rotary(O.matmul_nt_kernel_order(nx, w[0], n_mats=3), 2)
    xk = O.rotary(O.matmul_nt_kernel_order(nx, w[1], n_mats=3), 2)
    xv = O.matmul_nt_kernel_order(nx, w[2], n_mats=3)
    att = O.attention_prefill_kernel_order(xq, xk, xv, 2, 0)
    x = O.matmul_nt_kernel_order(att, w[3], beta=1.0, out=x)
    nx = O.rms_norm(x, fn, 1e-6)
    up = O.silu_mul(O.matmul_nt_kernel_order(nx, w[4], n_mats=2), O.matmul_nt_kernel_order(nx, w[6], n_mats=2))
    x = O.matmul_nt_kernel_order(up, w[5], beta=1.0, out=x)
    assert (x.view(np.uint16) == hid.view(np.uint16)).all()


def test_softmax_logits_kernel_order():
    for n, temp in ((32000, 0.8), (2048, 1.0), (8, 0.5)):
        x = f16(RNG.normal(0, 1.3, n))
        got = O.softmax_logits_kernel_order(x, temp)
        ref = O.softmax_rows(x.reshape(1, -1), temp)[0]
        # only the association of the sum differs: at most the last fp16 bit of a probability
        d = np.abs(got.view(np.uint16).astype(np.int32) - ref.view(np.uint16).astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= 0.02
        assert abs(got.astype(np.float64).sum() - 1.0) <= 2e-3
        assert np.argmax(got) == np.argmax(x)


# ------------------------------------------------------------------ rms norm
def test_rms_norm_closed_forms():
    cols = 512
    ones = np.ones(cols, dtype=np.float16)
    const = np.full((2, cols), 3.0, dtype=np.float16)
    const[1] = -0.25
    out = O.rms_norm(const, ones, 0.0)
    assert (out[0] == 1.0).all() and (out[1] == -1.0).all()
    x = f16(RNG.normal(0, 1, (7, cols)))
    w = f16(RNG.normal(1, 0.1, cols))
    out = O.rms_norm(x, w, 1e-6)
    x64 = x.astype(np.float64)
    inner = (x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6))
    ref = w.astype(np.float64) * inner
    assert rel_err(out, ref) < 2e-3  # two fp16 roundings
    # the two roundings happen in this order: fp16(x * rms_inv), then fp16(w * that)
    inner16 = inner.astype(np.float32).astype(np.float16)
    two_step = (w.astype(np.float32) * inner16.astype(np.float32)).astype(np.float16)
    assert (two_step.view(np.uint16) != out.view(np.uint16)).mean() < 0.01
    # scale invariance (eps = 0): norm(4x) == norm(x) exactly, powers of two commute with rounding
    assert (O.rms_norm(x * np.float16(4), w, 0.0).view(np.uint16) == O.rms_norm(x, w, 0.0).view(np.uint16)).all()


# ------------------------------------------------------------------ rotary
def test_rotary_properties():
    n_heads, head_dim = 4, 128
    dim = n_heads * head_dim
    x = f16(RNG.normal(0, 1, (6, dim)))
    r0 = O.rotary(x[:1], n_heads, pos_offset=0)
    assert (r0.view(np.uint16) == x[:1].view(np.uint16)).all()  # position 0 is the identity
    pos0 = 11
    out = O.rotary(x, n_heads, pos_offset=pos0).astype(np.float64)
    z = x.astype(np.float64).reshape(6, n_heads, head_dim // 2, 2)
    zc = z[..., 0] + 1j * z[..., 1]
    pos = (pos0 + np.arange(6))[:, None, None]
    freq = 1.0 / (10000.0 ** (np.arange(0, head_dim, 2) / head_dim))[None, None, :]
    ref = zc * np.exp(1j * pos * freq)
    got = out.reshape(6, n_heads, head_dim // 2, 2)
    gc = got[..., 0] + 1j * got[..., 1]
    assert np.max(np.abs(gc - ref)) < 4e-3  # fp32 angle at pos<=16 plus fp16 rounding
    assert np.max(np.abs(np.abs(gc) - np.abs(zc))) < 4e-3  # pair norm preserved
    # pair 0 of every head turns by exactly `pos` radians
    ang = np.angle(gc[:, :, 0] / zc[:, :, 0])
    want = np.angle(np.exp(1j * (pos0 + np.arange(6))))[:, None]
    assert np.max(np.abs(np.angle(np.exp(1j * (ang - want))))) < 5e-3


# ------------------------------------------------------------------ softmax
def test_softmax_properties():
    for w in (7, 256, 1000):
        u = np.full((3, w), 1.5, dtype=np.float16)
        out = O.softmax_rows(u)
        assert (out.view(np.uint16) == np.float16(np.float32(1.0) / np.float32(w)).view(np.uint16)).all()
    x = f16(RNG.normal(0, 2, (5, 777)))
    x[:, 400:] = -np.inf
    out = O.softmax_rows(x)
    assert (out[:, 400:] == 0).all()
    x64 = x[:, :400].astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(out[:, :400].astype(np.float64) - ref)) <= ref.max() * 2.0 ** -10
    assert np.all(np.abs(out.astype(np.float64).sum(axis=1) - 1) < 2e-3)
    # temperature divides the logits
    t = O.softmax_rows(x, temp=0.8)
    e = np.exp(x64 / np.float64(np.float32(0.8)) - (x64 / np.float64(np.float32(0.8))).max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(t[:, :400].astype(np.float64) - ref)) <= ref.max() * 2.0 ** -10
    # 3-d input: every leading index is a row
    y = f16(RNG.normal(0, 1, (2, 3, 50)))
    assert (O.softmax_rows(y).reshape(6, 50).view(np.uint16) == O.softmax_rows(y.reshape(6, 50)).view(np.uint16)).all()


# ------------------------------------------------------------------ attention
def np_attention64(q, k, v, n_heads, start_pos):
    n, dim = q.shape
    T = k.shape[0]
    hd = dim // n_heads
    out = np.zeros((n, dim))
    for h in range(n_heads):
        qs, ks, vs = (a[:, h * hd:(h + 1) * hd].astype(np.float64) for a in (q, k, v))
        s = qs @ ks.T / np.sqrt(hd)
        mask = np.arange(T)[None, :] > (np.arange(n)[:, None] + start_pos)
        s[mask] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, h * hd:(h + 1) * hd] = p @ vs
    return out


@pytest.mark.parametrize("n,T,start", [(5, 5, 0), (1, 9, 8), (3, 10, 7)])
def test_attention_vs_float64(n, T, start):
    n_heads, hd = 3, 32
    dim = n_heads * hd
    q = f16(RNG.normal(0, 1, (n, dim)))
    k = f16(RNG.normal(0, 1, (T, dim)))
    v = f16(RNG.normal(0, 1, (T, dim)))
    out = O.attention(q, k, v, n_heads, start)
    ref = np_attention64(q, k, v, n_heads, start)
    assert np.max(np.abs(out.astype(np.float64) - ref)) < 4e-3
    s = O.matmul_qk(q, k, n_heads, start)
    assert s.shape == (n_heads, n, T)
    for r in range(n):
        assert np.isneginf(s[:, r, r + start + 1:]).all() and np.isfinite(s[:, r, :r + start + 1]).all()
    # the 1/sqrt(head_dim) scale and the head slicing
    h = 2
    want = q[0, h * hd:(h + 1) * hd].astype(np.float64) @ k[0, h * hd:(h + 1) * hd].astype(np.float64) / np.sqrt(hd)
    assert abs(float(s[h, 0, 0]) - want) <= abs(want) * 2.0 ** -10 + 1e-6


def test_attention_first_row_is_v0():
    n_heads, hd, n = 2, 64, 4
    dim = n_heads * hd
    q, k, v = (f16(RNG.normal(0, 1, (n, dim))) for _ in range(3))
    out = O.attention(q, k, v, n_heads, 0)
    assert (out[0].view(np.uint16) == v[0].view(np.uint16)).all()  # causal row 0 sees only itself, p = 1


def test_decode_equals_last_prefill_row():
    n_heads, hd, T = 2, 64, 12
    dim = n_heads * hd
    q, k, v = (f16(RNG.normal(0, 1, (T, dim))) for _ in range(3))
    full = O.attention(q, k, v, n_heads, 0)
    last = O.attention(q[-1:], k, v, n_heads, T - 1)
    assert (full[-1:].view(np.uint16) == last.view(np.uint16)).all()


# ------------------------------------------------------------------ silu, embed, argmax
def test_silu_mul():
    a = f16(RNG.normal(0, 2, 5000))
    b = f16(RNG.normal(0, 1, 5000))
    out = O.silu_mul(a, b)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    ref = a64 / (1 + np.exp(-a64)) * b64
    assert np.max(np.abs(out.astype(np.float64) - ref)) <= np.max(np.abs(ref)) * 2.0 ** -10
    z = O.silu_mul(np.zeros(4, dtype=np.float16), b[:4])
    assert (z == 0).all()
    big = O.silu_mul(np.array([20.0, -20.0], dtype=np.float16), np.array([1.0, 1.0], dtype=np.float16))
    assert big[0] == 20.0 and abs(float(big[1])) < 1e-6


def test_embed_and_embed_u8():
    table = f16(RNG.normal(0, 0.02, (50, 256)))
    ids = [3, 49, 0, 3]
    out = O.embed(ids, table)
    assert (out.view(np.uint16) == table[ids].view(np.uint16)).all()
    codes, scales = O.quantize_absmax_u8(table, 128)
    out8 = O.embed_u8(ids, codes, scales, 128)
    assert (out8.view(np.uint16) == O.dequantize_absmax_u8(codes, scales, 128)[ids].view(np.uint16)).all()


def test_argmax_first_wins():
    p = np.array([0.1, 0.5, 0.2, 0.5, 0.5], dtype=np.float16)
    assert O.argmax_first(p) == 1
    assert O.argmax_first(np.array([0.0, -0.0], dtype=np.float16)) == 0
    assert O.argmax_first(np.array([1, 2, 3], dtype=np.float16)) == 2


# ------------------------------------------------------------------ error_stats (transform.cu:99-150)
def test_error_stats_closed_forms():
    a = f16(RNG.normal(0, 1, 10000))
    assert (O.error_stats(a, a) == 0).all()
    # a constant offset that fp16 represents exactly: every difference is 0.5
    b = f16(np.arange(1000) * 0.5)
    c = f16(np.arange(1000) * 0.5 + 0.5)
    assert np.allclose(O.error_stats(c, b), [0.25, 0.5, 0.5], rtol=0, atol=0)
    # one differing element among n: mse = d^2 / n, max = d, mean abs = d / n
    d = a.copy()
    d[1234] = np.float16(float(a[1234]) + 2.0)
    delta = abs(float(d[1234]) - float(a[1234]))
    mse, mx, mean = O.error_stats(d, a)
    assert mx == np.float32(delta)
    assert np.isclose(mse, delta * delta / a.size, rtol=1e-6) and np.isclose(mean, delta / a.size, rtol=1e-6)
    # against float64 numpy on random data; sign of the difference must not matter
    e = f16(RNG.normal(0, 1, 10000))
    diff = a.astype(np.float32) - e.astype(np.float32)
    want = [np.mean(diff.astype(np.float64) ** 2), np.max(np.abs(diff)), np.mean(np.abs(diff.astype(np.float64)))]
    assert np.allclose(O.error_stats(a, e), want, rtol=1e-6)
    assert np.allclose(O.error_stats(e, a), want, rtol=1e-6)


def test_sample_row_closed_forms():
    # one-hot row: that index for every random number
    p = np.zeros(100, dtype=np.float16)
    p[37] = 1.0
    for r in (0, 1, 2**63, 2**64 - 1):
        assert O.sample_row(p, r) == 37
    # weights 1 : 3 -> index 0 exactly while random < 2^62 (r = floor(random * total / 2^64) < weight 0)
    p = np.array([0.25, 0.75], dtype=np.float16)
    assert O.sample_row(p, 2**62 - 1) == 0
    assert O.sample_row(p, 2**62) == 1
    assert O.sample_row(p, 2**64 - 1) == 1
    # zero, negative and NaN entries are never drawn; the smallest subnormal (2^-24, weight 1) can be
    p = np.array([0.0, -1.0, np.nan, 2.0**-24, 0.0, 2.0**-24], dtype=np.float16)
    seen = {O.sample_row(p, r) for r in range(0, 2**64, 2**64 // 64)}
    assert seen == {3, 5}
    assert O.sample_row(p, 2**63 - 1) == 3 and O.sample_row(p, 2**63) == 5
    # nothing to draw from: index 0
    assert O.sample_row(np.zeros(10, dtype=np.float16), 12345) == 0
    # monotone in the random number, and every index of a uniform row is reached in order
    p = np.full(8, 0.125, dtype=np.float16)
    idx = [O.sample_row(p, r) for r in range(0, 2**64, 2**64 // 1024)]
    assert idx == sorted(idx) and [idx.count(k) for k in range(8)] == [128] * 8


def test_sample_row_frequencies():
    # frequencies over the step-random sequence follow p / sum(p) (here sum(p) != 1 on purpose)
    rng = np.random.default_rng(5)
    p = rng.random(50).astype(np.float16) * np.float16(0.04)
    w = p.astype(np.float64) / p.astype(np.float64).sum()
    n = 20000
    counts = np.bincount([O.sample_row(p, O.step_random(99, k)) for k in range(n)], minlength=50)
    # five standard deviations of a binomial count, per index
    assert (np.abs(counts - n * w) <= 5 * np.sqrt(n * w * (1 - w)) + 1).all()


def test_step_random_is_splitmix64():
    # reference values of the splitmix64 generator seeded with 1234567 (Vigna's test vector)
    expect = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    assert [O.step_random(1234567, k) for k in range(5)] == expect
