"""GPU parity of every kernel behind the C ABI against the CPU oracle, on the same seeded inputs.

Bars: bit-exact for the quantiser's codes and scales, for dequantisation, embedding, RoPE and the
argmax; max-abs-rel <= 1e-2 for every fp16 output that accumulates in fp32 (matmul, attention,
softmax, norm, silu)."""
import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max-abs-rel bar for fp16 outputs with fp32 accumulation


@pytest.fixture(scope="module", autouse=True)
def gpu():
    import gpu_helpers as G
    G.setup()
    yield G
    G.release()


def normal(shape, seed, stream, std):
    n = int(np.prod(shape))
    return O.fill_normal_f16(n, seed, stream, std).reshape(shape)


def test_fill_normal_matches_oracle_bits(gpu):
    G = gpu
    for n, seed, stream, std in [(1000, 0, 1, 0.02), (1 << 20, 7, 33, 1.0), (12345, 2 ** 40 + 3, 2 ** 33, 0.5)]:
        buf = G.empty((n,))
        G.B.check(G.L().lcu_fill_normal_f16(buf.ptr, n, seed, stream, std, None))
        got = G.host(buf, (n,))
        assert (got.view(np.uint16) == O.fill_normal_f16(n, seed, stream, std).view(np.uint16)).all()


@pytest.mark.parametrize("rows,cols,block", [(64, 1024, 128), (7, 512, 32), (5, 2048, 1024), (33, 768, 256)])
def test_quantize_bit_exact(gpu, rows, cols, block):
    G = gpu
    w = normal((rows, cols), 3, 5, 0.02)
    w[0, :block] = 0  # an all-zero block
    w[1, 3] = np.float16(65504.0)
    w[2, :block] = np.float16(6e-8)  # scale underflows to zero
    codes_d, scales_d = G.empty((rows, cols), np.uint8), G.empty((rows, cols // block))
    wd = G.dev(w)
    G.B.check(G.L().lcu_quantize_absmax_u8(codes_d.ptr, scales_d.ptr, wd.ptr, rows, cols, block, None))
    codes, scales = G.host(codes_d, (rows, cols), np.uint8), G.host(scales_d, (rows, cols // block))
    ec, es = O.quantize_absmax_u8(w, block)
    assert (scales.view(np.uint16) == es.view(np.uint16)).all()
    assert (codes == ec).all()
    out_d = G.empty((rows, cols))
    G.B.check(G.L().lcu_dequantize_absmax_u8(out_d.ptr, scales_d.ptr, codes_d.ptr, rows, cols, block, None))
    assert (G.host(out_d, (rows, cols)).view(np.uint16) == O.dequantize_absmax_u8(ec, es, block).view(np.uint16)).all()


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_quantize_bit_exact_at_llama7b_shapes(gpu, rows, cols):
    """the weight matrices of the int8 benchmark configuration, W ~ N(0, 0.02), block 128: every code and scale"""
    G = gpu
    x = normal((rows, cols), 0, 310, 0.02)
    codes_d, scales_d = G.empty((rows, cols), np.uint8), G.empty((rows, cols // 128))
    G.B.check(G.L().lcu_quantize_absmax_u8(codes_d.ptr, scales_d.ptr, G.dev_keep(x).ptr, rows, cols, 128, None))
    ec, es = O.quantize_absmax_u8(x, 128)
    assert (G.host(codes_d, (rows, cols), np.uint8) == ec).all()
    assert (G.host(scales_d, (rows, cols // 128)).view(np.uint16) == es.view(np.uint16)).all()
    back_d = G.empty((rows, cols))
    G.B.check(G.L().lcu_dequantize_absmax_u8(back_d.ptr, scales_d.ptr, codes_d.ptr, rows, cols, 128, None))
    assert (G.host(back_d, (rows, cols)).view(np.uint16) == O.dequantize_absmax_u8(ec, es, 128).view(np.uint16)).all()
    G.release()


def test_quantize_exhaustive_inputs_bit_exact(gpu):
    G = gpu
    allbits = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = allbits[np.isfinite(allbits)]
    for absmax in [np.float16(65504.0), np.float16(1.0), np.float16(0.0604), np.float16(3e-4)]:
        xs = finite[np.abs(finite) <= absmax]
        n = (len(xs) + 126) // 127
        blocks = np.zeros((n, 128), dtype=np.float16)
        blocks[:, 0] = absmax
        flat = np.zeros(n * 127, dtype=np.float16)
        flat[: len(xs)] = xs
        blocks[:, 1:] = flat.reshape(n, 127)
        codes_d, scales_d = G.empty((n, 128), np.uint8), G.empty((n, 1))
        G.B.check(G.L().lcu_quantize_absmax_u8(codes_d.ptr, scales_d.ptr, G.dev_keep(blocks).ptr, n, 128, 128, None))
        ec, es = O.quantize_absmax_u8(blocks, 128)
        assert (G.host(codes_d, (n, 128), np.uint8) == ec).all()
        assert (G.host(scales_d, (n, 1)).view(np.uint16) == es.view(np.uint16)).all()


def test_dequantize_all_codes_all_scales_bit_exact(gpu):
    G = gpu
    # every code against a sweep of scales including subnormal ones
    scales = np.concatenate([np.arange(0, 0x0500, 7, dtype=np.uint16), np.arange(0x0500, 0x5C00, 97, dtype=np.uint16)])
    scales = scales.view(np.float16).reshape(-1, 1)
    n = len(scales)
    codes = np.tile(np.arange(256, dtype=np.uint8), (n, 1))
    out_d = G.empty((n, 256))
    G.B.check(G.L().lcu_dequantize_absmax_u8(out_d.ptr, G.dev_keep(scales).ptr, G.dev_keep(codes).ptr, n, 256, 256, None))
    assert (G.host(out_d, (n, 256)).view(np.uint16) == O.dequantize_absmax_u8(codes, scales, 256).view(np.uint16)).all()


GEMV_SHAPES = [(4096, 11008), (4096, 4096), (11008, 4096), (256, 40), (1032, 77), (6656, 6656)]


@pytest.mark.parametrize("K,N", GEMV_SHAPES)
def test_gemv_f16(gpu, K, N):
    G = gpu
    x = normal((1, K), 0, 100, 1.0)
    w = normal((N, K), 0, 101, 0.02)
    got = G.gemm_f16(x, w)
    ref = O.matmul_nt(x, w)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05  # same fp16 value except where fp32 summation order flips a rounding
    # against the oracle's restatement of this kernel's own summation order: every bit
    assert G.ulp_mismatch(got, O.matmul_nt(x, w, flavour=2)) == 0.0
    old = normal((1, N), 0, 102, 1.0)
    got = G.gemm_f16(x, w, beta=1.0, out=old)
    assert G.max_abs_rel(got, O.matmul_nt(x, w, beta=1.0, out=old)) <= TOL
    assert G.ulp_mismatch(got, O.matmul_nt(x, w, beta=1.0, out=old, flavour=2)) == 0.0
    G.release()


def test_gemv_exact_cases(gpu):
    G = gpu
    K = 512
    x = normal((1, K), 1, 1, 1.0)
    assert (G.gemm_f16(x, np.eye(K, dtype=np.float16)).view(np.uint16) == x.view(np.uint16)).all()
    w = normal((300, K), 1, 2, 0.02)
    onehot = np.zeros((1, K), dtype=np.float16)
    onehot[0, 129] = 1
    assert (G.gemm_f16(onehot, w)[0].view(np.uint16) == w[:, 129].view(np.uint16)).all()
    G.release()


# rows of one to six batches of the workgroup (4096 codes each): two to five are requested at once, one
# and six go through the loop; two and four rows per workgroup (N below / from 6144)
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 11008), (11008, 4096), (256, 40), (1024 + 128, 77), (6656, 17920),
                                 (17920, 300), (13824, 100), (22016, 64), (8192, 6200), (17920, 6152)])
def test_gemv_u8(gpu, K, N):
    G = gpu
    x = normal((1, K), 0, 200, 1.0)
    w = normal((N, K), 0, 201, 0.02)
    codes, scales = O.quantize_absmax_u8(w, 128)
    got = G.gemm_u8(x, codes, scales, 128)
    ref = O.matmul_nt_u8(x, codes, scales, 128)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05
    # the kernel-order flavour restates the kernel's sums down to the alignment inside
    # v_dot2_f32_f16: every output bit for bit
    assert G.ulp_mismatch(got, O.matmul_nt_u8(x, codes, scales, 128, flavour=2)) == 0.0
    old = normal((1, N), 0, 202, 1.0)
    got = G.gemm_u8(x, codes, scales, 128, beta=1.0, out=old)
    assert G.max_abs_rel(got, O.matmul_nt_u8(x, codes, scales, 128, beta=1.0, out=old)) <= TOL
    assert G.ulp_mismatch(got, O.matmul_nt_u8(x, codes, scales, 128, beta=1.0, out=old, flavour=2)) == 0.0
    G.release()


def test_gemv_u8_dequant_is_exact(gpu):
    # one-hot x picks single dequantised weights: they must be the reference's fp16 values exactly
    G = gpu
    K, N = 256, 64
    w = normal((N, K), 4, 1, 0.02)
    w[:, 128:] *= np.float16(1e-3)  # small scales, some products subnormal in fp16
    codes, scales = O.quantize_absmax_u8(w, 128)
    deq = O.dequantize_absmax_u8(codes, scales, 128)
    for k in (0, 5, 127, 128, 200, 255):
        x = np.zeros((1, K), dtype=np.float16)
        x[0, k] = 1
        got = G.gemm_u8(x, codes, scales, 128)[0]
        assert (got.view(np.uint16) == deq[:, k].view(np.uint16)).all(), k
    G.release()


# the shapes cover every tile configuration of the dispatcher: 128x64 with two wavefront groups,
# 256x128, 128x128 with eight wavefronts (160..255 tiles: N = 5120), 128x64 with two workgroups per
# compute unit (N = 4160), 128x128 with four wavefronts (M = 1024, N = 4096), ragged K / M / N, and
# grids with more tiles than the chip holds workgroups at once ((4096, 128, 4096) .. (2100, 128, 8200)); the
# last five are short prompts (2..64 rows), which split K over several workgroups per tile: 32- and 64-row
# tiles, uneven splits (11008 / 64 = 172 stages over 16 workgroups), ragged M and N
@pytest.mark.parametrize("M,K,N", [(512, 4096, 4096), (512, 4096, 11008), (512, 11008, 4096), (128, 256, 128),
                                   (7, 64, 24), (130, 200, 70), (33, 1024, 257), (512, 256, 5120), (512, 384, 4160),
                                   (1024, 256, 4096), (500, 128, 5100), (4096, 128, 4096), (512, 256, 17920), (2100, 128, 8200),
                                   (2, 4096, 4096), (17, 1024, 5000), (32, 11008, 4096), (33, 1024, 4100), (64, 4096, 11008)])
def test_gemm_f16(gpu, M, K, N):
    G = gpu
    x = normal((M, K), 0, 300, 1.0)
    w = normal((N, K), 0, 301, 0.02)
    got = G.gemm_f16(x, w)
    ref = O.matmul_nt(x, w)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05
    # the kernel-order flavour restates the matrix cores' sums and the dispatcher's cut of K: bit for bit
    assert G.ulp_mismatch(got, O.matmul_nt(x, w, flavour=2)) == 0.0, O.gemm_plan(M, K, N)
    old = normal((M, N), 0, 302, 1.0)
    got = G.gemm_f16(x, w, beta=1.0, out=old)
    assert G.max_abs_rel(got, O.matmul_nt(x, w, beta=1.0, out=old)) <= TOL
    assert G.ulp_mismatch(got, O.matmul_nt(x, w, beta=1.0, out=old, flavour=2)) == 0.0
    G.release()


def test_gemm_residual_into_an_output_that_is_not_16_byte_aligned(gpu):
    """beta = 1 with the output tile 8 bytes off a 16-byte boundary: the tile that fetches its old values in 16-byte
    pieces (512 x 4096 x 4096, the Wo product) must fall back to 2-byte reads; same bits as the aligned call."""
    G = gpu
    M, K, N = 512, 4096, 4096
    x = normal((M, K), 0, 310, 1.0)
    w = normal((N, K), 0, 311, 0.02)
    old = normal((M, N), 0, 312, 1.0)
    want = G.gemm_f16(x, w, beta=1.0, out=old)
    buf = G.empty((M * N + 8,))
    for shift in (4, 1):  # halves: 8 bytes and 2 bytes off
        padded = np.zeros(M * N + 8, dtype=np.float16)
        padded[shift:shift + M * N] = old.reshape(-1)
        G.B.check(G.L().lcu_h2d(buf.ptr, padded.ctypes.data, padded.nbytes, None))
        G.B.check(G.L().lcu_gemm_f16_nt(buf.ptr + 2 * shift, G.dev_keep(x).ptr, G.dev_keep(w).ptr, M, K, N, 1.0, None))
        got = G.host(buf, (M * N + 8,))[shift:shift + M * N].reshape(M, N)
        assert (got.view(np.uint16) == want.view(np.uint16)).all(), shift
    buf.free()
    G.release()


def test_gemm_exact_cases(gpu):
    G = gpu
    K = 256
    x = normal((40, K), 2, 1, 1.0)
    assert (G.gemm_f16(x, np.eye(K, dtype=np.float16)).view(np.uint16) == x.view(np.uint16)).all()
    # asymmetric operands: out[m, n] pairs lhs row m with rhs row n
    w = np.zeros((96, K), dtype=np.float16)
    w[70, 5] = 2
    x2 = np.zeros((40, K), dtype=np.float16)
    x2[33, 5] = 3
    out = G.gemm_f16(x2, w)
    assert out[33, 70] == 6 and np.count_nonzero(out) == 1
    G.release()


@pytest.mark.parametrize("M,K,N", [(512, 4096, 4096), (512, 4096, 11008), (512, 11008, 4096), (16, 256, 128),
                                   (130, 384, 70), (512, 256, 5120), (512, 384, 4160), (1024, 256, 4096),
                                   (500, 128, 5100), (40, 384, 300), (4096, 128, 4096), (512, 256, 17920),
                                   (5, 4096, 4096), (17, 1024, 5000), (32, 11008, 4096), (64, 1024, 4100), (512, 17920, 6656)])
def test_gemm_u8(gpu, M, K, N):
    G = gpu
    x = normal((M, K), 0, 400, 1.0)
    w = normal((N, K), 0, 401, 0.02)
    codes, scales = O.quantize_absmax_u8(w, 128)
    got = G.gemm_u8(x, codes, scales, 128)
    ref = O.matmul_nt_u8(x, codes, scales, 128)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05
    assert G.ulp_mismatch(got, O.matmul_nt_u8(x, codes, scales, 128, flavour=2)) == 0.0, O.gemm_plan(M, K, N, True)
    # row r of the M-row product equals the single-row product (decode path) within tolerance
    one = G.gemm_u8(x[3:4], codes, scales, 128)
    assert G.max_abs_rel(one, got[3:4]) <= TOL
    G.release()


@pytest.mark.parametrize("M,K,N,count", [(512, 512, 4096, 3), (8, 4096, 4096, 3), (40, 1024, 11008, 2), (300, 256, 700, 2),
                                          (33, 200, 70, 3), (1, 512, 300, 3)])
def test_gemm_multi_matches_separate_calls(gpu, M, K, N, count):
    """Several weight matrices of one shape in one launch (Wq, Wk, Wv; W1, W3): what separate calls give
    (to the matmul tolerance: the fused launch may pick another tile shape, hence another summation order)
    and what the oracle gives, for fp16 and uint8 weights, in every dispatch branch (large tiles,
    short-prompt split-K, ragged K, a single row)."""
    G = gpu
    L = G.L()
    VP = G.B.vp
    x = normal((M, K), 0, 1600, 1.0)
    xd = G.dev_keep(x)
    ws = [normal((N, K), 0, 1601 + g, 0.02) for g in range(count)]
    wd = [G.dev_keep(w) for w in ws]
    sep = [G.gemm_f16(x, w) for w in ws]
    outs = [G.empty((M, N)) for _ in range(count)]
    out_arr = (VP * count)(*[o.ptr for o in outs])
    w_arr = (VP * count)(*[w.ptr for w in wd])
    G.B.check(L.lcu_gemm_f16_nt_multi(out_arr, xd.ptr, w_arr, count, M, K, N, 0.0, None))
    for g in range(count):
        got = G.host(outs[g], (M, N))
        assert G.max_abs_rel(got, sep[g]) <= TOL and G.ulp_mismatch(got, sep[g]) < 0.05, g
        assert G.max_abs_rel(got, O.matmul_nt(x, ws[g])) <= TOL, g
        if K % 8 == 0:
            assert G.ulp_mismatch(got, O.matmul_nt_kernel_order(x, ws[g], n_mats=count)) == 0.0, g
    if K % 128 == 0:
        q = [O.quantize_absmax_u8(w, 128) for w in ws]
        cd = [G.dev_keep(c) for c, _ in q]
        sd = [G.dev_keep(sc) for _, sc in q]
        sep = [G.gemm_u8(x, c, sc, 128) for c, sc in q]
        c_arr = (VP * count)(*[c.ptr for c in cd])
        s_arr = (VP * count)(*[sc.ptr for sc in sd])
        G.B.check(L.lcu_gemm_f16u8_nt_multi(out_arr, xd.ptr, c_arr, s_arr, count, M, K, N, 128, 0.0, None))
        for g in range(count):
            got = G.host(outs[g], (M, N))
            assert G.max_abs_rel(got, sep[g]) <= TOL and G.ulp_mismatch(got, sep[g]) < 0.05, g
            assert G.max_abs_rel(got, O.matmul_nt_u8(x, q[g][0], q[g][1], 128)) <= TOL, g
            assert G.ulp_mismatch(got, O.matmul_nt_kernel_order(x, codes=q[g][0], scales=q[g][1], block=128,
                                                               n_mats=count)) == 0.0, g
    # beta = 1: every output starts from its own earlier contents
    olds = [normal((M, N), 0, 1650 + g, 1.0) for g in range(count)]
    for g in range(count):
        G.B.check(L.lcu_h2d(outs[g].ptr, olds[g].ctypes.data_as(VP), olds[g].nbytes, None))
    G.B.check(L.lcu_gemm_f16_nt_multi(out_arr, xd.ptr, w_arr, count, M, K, N, 1.0, None))
    for g in range(count):
        assert G.max_abs_rel(G.host(outs[g], (M, N)), O.matmul_nt(x, ws[g], beta=1.0, out=olds[g])) <= TOL, g
    assert L.lcu_gemm_f16_nt_multi(out_arr, xd.ptr, w_arr, 4, M, K, N, 0.0, None) == -2
    G.release()


def test_gemm_dispatch_sweep_bit_exact(gpu):
    """Seventy seeded shapes across the dispatcher's branches (few and many rows, K in whole stages or
    ragged, tile counts on both sides of every threshold, one to three matrices per launch, fp16 and
    uint8): the oracle's restatement of the cut of K must give the device's bits on all of them."""
    G = gpu
    L = G.L()
    VP = G.B.vp
    rng = np.random.default_rng(77)
    plans = set()
    for case in range(70):
        M = int(rng.choice([2, 7, 32, 33, 64, 65, 100, 256, 300, 512, 700, 1100]))
        K = int(rng.choice([64, 128, 136, 256, 384, 640, 1024, 2560, 5120]))
        N = int(rng.choice([24, 128, 1000, 2048, 4096, 5120, 8200, 11008, 17920]))
        nm = int(rng.choice([1, 1, 2, 3]))
        u8 = bool(rng.integers(0, 2)) and K % 128 == 0
        if M * K * N * nm > 2.5e10:
            K = 128
        x = normal((M, K), 5, 3 * case, 1.0)
        ws = [normal((N, K), 5, 3 * case + 1 + g, 0.02) for g in range(nm)]
        xd = G.dev_keep(x)
        outs = [G.empty((M, N)) for _ in range(nm)]
        out_arr = (VP * nm)(*[o.ptr for o in outs])
        if u8:
            q = [O.quantize_absmax_u8(w, 128) for w in ws]
            cd, sd = [G.dev_keep(c) for c, _ in q], [G.dev_keep(sc) for _, sc in q]
            G.B.check(L.lcu_gemm_f16u8_nt_multi(out_arr, xd.ptr, (VP * nm)(*[c.ptr for c in cd]), (VP * nm)(*[sc.ptr for sc in sd]),
                                                nm, M, K, N, 128, 0.0, None))
            want = [O.matmul_nt_kernel_order(x, codes=c, scales=sc, block=128, n_mats=nm) for c, sc in q]
        else:
            wd = [G.dev_keep(w) for w in ws]
            G.B.check(L.lcu_gemm_f16_nt_multi(out_arr, xd.ptr, (VP * nm)(*[w.ptr for w in wd]), nm, M, K, N, 0.0, None))
            want = [O.matmul_nt_kernel_order(x, w, n_mats=nm) for w in ws]
        plan = O.gemm_plan(M, K, N, u8, 128, nm)
        plans.add(plan)
        for g in range(nm):
            assert G.ulp_mismatch(G.host(outs[g], (M, N)), want[g]) == 0.0, (case, M, K, N, nm, u8, plan, g)
        G.release()
    assert len(plans) >= 6, plans  # single chains, two groups per stage, several depths of split


def test_streams_own_their_workspace(gpu):
    """Split-K products (2..64 rows) keep fp32 partial sums in scratch memory.  Every stream made by
    lcu_stream_create has a workspace of its own, so two host threads driving two streams at once
    get the results of a single undisturbed call, bit for bit."""
    import ctypes as C
    import threading
    G = gpu
    L = G.L()
    K, N = 4096, 4096
    cases = []
    for t in range(2):
        x = normal((8 + 8 * t, K), 3, 40 + t, 1.0)
        w = normal((N, K), 3, 50 + t, 0.02)
        cases.append((x, w, G.gemm_f16(x, w)))
    G.release()
    results = [None, None]

    def work(t):
        x, w, _ = cases[t]
        stream = G.B.vp()
        G.B.check(L.lcu_stream_create(C.byref(stream)))
        xd, wd, od = G.dev(x), G.dev(w), G.empty((x.shape[0], N))
        bad = 0
        for _ in range(200):
            G.B.check(L.lcu_gemm_f16_nt(od.ptr, xd.ptr, wd.ptr, x.shape[0], K, N, 0.0, stream))
        G.B.check(L.lcu_sync(stream))
        results[t] = G.host(od, (x.shape[0], N))
        G.B.check(L.lcu_stream_destroy(stream))
        for b in (xd, wd, od):
            b.free()

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    for t in range(2):
        assert results[t] is not None and (results[t].view(np.uint16) == cases[t][2].view(np.uint16)).all()


def test_gemm_rejects_bad_shapes(gpu):
    G = gpu
    a = G.dev(np.zeros((4, 12), dtype=np.float16))
    assert G.L().lcu_gemm_f16_nt(a.ptr, a.ptr, a.ptr, 4, 12, 4, 0.0, None) == -2  # K % 8
    assert G.L().lcu_gemm_f16_nt(None, a.ptr, a.ptr, 4, 16, 4, 0.0, None) == -2
    assert G.L().lcu_gemm_f16u8_nt(a.ptr, a.ptr, a.ptr, a.ptr, 1, 256, 4, 100, 0.0, None) == -2
    assert b"lcu_gemm_f16u8_nt" in G.L().lcu_last_error()
    assert G.L().lcu_gemm_f16_nt(a.ptr, a.ptr, a.ptr, 0, 16, 4, 0.0, None) == 0  # empty input is fine


@pytest.mark.parametrize("rows,cols", [(1, 4096), (512, 4096), (3, 6656), (5, 200)])
def test_rmsnorm(gpu, rows, cols):
    G = gpu
    x = normal((rows, cols), 0, 500, 1.0)
    w = (normal((cols,), 0, 501, 0.1).astype(np.float32) + 1).astype(np.float16)
    out_d = G.empty((rows, cols))
    G.B.check(G.L().lcu_rmsnorm(out_d.ptr, G.dev_keep(x).ptr, G.dev_keep(w).ptr, rows, cols, 1e-6, None))
    got = G.host(out_d, (rows, cols))
    ref = O.rms_norm(x, w, 1e-6)
    assert G.max_abs_rel(got, ref) <= TOL
    # same reduction order and IEEE 1/sqrt on both sides
    assert G.ulp_mismatch(got, ref) == 0.0
    G.release()


@pytest.mark.parametrize("rows,pos", [(1, 0), (1, 1337), (512, 0), (40, 2000)])
def test_rope_bit_exact(gpu, rows, pos):
    G = gpu
    heads, dim = 32, 4096
    x = normal((rows, dim), 0, 600, 1.0)
    tab = G.B.vp()
    G.B.check(G.L().lcu_rope_table_create(G.B.C.byref(tab), 2048, 128, 10000.0))
    out_d = G.empty((rows, dim))
    G.B.check(G.L().lcu_rope(out_d.ptr, G.dev_keep(x).ptr, rows, dim, heads, pos, tab, 2048, None))
    got = G.host(out_d, (rows, dim))
    assert G.ulp_mismatch(got, O.rotary(x, heads, pos_offset=pos)) == 0.0
    # in place
    xd = G.dev(x)
    G.B.check(G.L().lcu_rope(xd.ptr, xd.ptr, rows, dim, heads, pos, tab, 2048, None))
    assert G.ulp_mismatch(G.host(xd, (rows, dim)), got) == 0.0
    assert G.L().lcu_rope(xd.ptr, xd.ptr, rows, dim, heads, 2048 - rows + 1, tab, 2048, None) == -2  # past the table
    # two tensors in one launch
    y = normal((rows, dim), 0, 601, 1.0)
    ad, bd = G.dev(x), G.dev(y)
    G.B.check(G.L().lcu_rope_pair(ad.ptr, bd.ptr, rows, dim, heads, pos, tab, 2048, None))
    assert G.ulp_mismatch(G.host(ad, (rows, dim)), got) == 0.0
    assert G.ulp_mismatch(G.host(bd, (rows, dim)), O.rotary(y, heads, pos_offset=pos)) == 0.0
    assert G.L().lcu_rope_pair(ad.ptr, bd.ptr, rows, dim, heads, 2048 - rows + 1, tab, 2048, None) == -2
    G.release()
    G.L().lcu_free(tab)


@pytest.mark.parametrize("rows,w,temp", [(1, 32000, 0.8), (64, 512, 1.0), (3, 77, 1.0), (2, 2048, 0.9)])
def test_softmax_rows(gpu, rows, w, temp):
    G = gpu
    x = normal((rows, w), 0, 700, 2.0)
    if w > 100:
        x[:, w - 30:] = -np.inf
    out_d = G.empty((rows, w))
    G.B.check(G.L().lcu_softmax_rows(out_d.ptr, G.dev_keep(x).ptr, rows, w, temp, None))
    got = G.host(out_d, (rows, w))
    ref = O.softmax_rows(x, temp)
    assert G.ulp_mismatch(got, ref) == 0.0  # same association of the sums, same exponential: every bit
    if w > 100:
        assert (got[:, w - 30:] == 0).all()
    G.release()


def test_silu_mul(gpu):
    G = gpu
    n = 512 * 11008
    a, b = normal((n,), 0, 800, 2.0), normal((n,), 0, 801, 1.0)
    out_d = G.empty((n,))
    G.B.check(G.L().lcu_silu_mul(out_d.ptr, G.dev_keep(a).ptr, G.dev_keep(b).ptr, n, None))
    got = G.host(out_d, (n,))
    ref = O.silu_mul(a, b)
    assert G.ulp_mismatch(got, ref) == 0.0
    # ragged length (the last thread's eight elements are cut) and buffers off the 16-byte grid
    for n2, off in ((2051, 0), (1000, 3)):
        ad, bd, od = G.dev_keep(a[:n2 + off]), G.dev_keep(b[:n2 + off]), G.empty((n2 + off,))
        G.B.check(G.L().lcu_silu_mul(od.ptr + 2 * off, ad.ptr + 2 * off, bd.ptr + 2 * off, n2, None))
        got2 = G.host(od, (n2 + off,))[off:]
        assert (got2.view(np.uint16) == got[off:n2 + off].view(np.uint16)).all()
    G.release()


def test_exp_bit_exact(gpu):
    """the exponential of every softmax and SiLU: host restatement and kernel agree on every bit"""
    G = gpu
    rng = np.random.default_rng(5)
    x = np.concatenate([np.linspace(-100, 95, 1 << 20), rng.normal(0, 4, 1 << 20), rng.uniform(-18, 0, 1 << 20),
                        [0.0, -0.0, np.inf, -np.inf, 88.72283, 88.72284, -87.33654, -87.33655, -87.3]]).astype(np.float32)
    out_d = G.B.empty(x.shape, np.float32)
    G.B.check(G.L().lcu_exp_f32(out_d.ptr, G.dev_keep(x).ptr, x.size, None))
    got = G.host(out_d, x.shape, np.float32)
    assert (got.view(np.uint32) == O.exp_f32(x).view(np.uint32)).all()
    G.release()


def test_embed_bit_exact(gpu):
    G = gpu
    vocab, dim = 1000, 512
    table = normal((vocab, dim), 0, 900, 0.02)
    ids = np.array([0, 999, 5, 5, 123], dtype=np.int16)
    out_d = G.empty((len(ids), dim))
    G.B.check(G.L().lcu_embed(out_d.ptr, G.dev_keep(ids).ptr, len(ids), dim, G.dev_keep(table).ptr, vocab, None))
    assert G.ulp_mismatch(G.host(out_d, (len(ids), dim)), O.embed(ids, table)) == 0.0
    codes, scales = O.quantize_absmax_u8(table, 128)
    G.B.check(G.L().lcu_embed_u8(out_d.ptr, G.dev_keep(ids).ptr, len(ids), dim, G.dev_keep(codes).ptr,
                                 G.dev_keep(scales).ptr, 128, vocab, None))
    assert G.ulp_mismatch(G.host(out_d, (len(ids), dim)), O.embed_u8(ids, codes, scales, 128)) == 0.0
    # an id outside the table gives zeros, not a stray read
    bad = np.array([1000, -1], dtype=np.int16)
    G.B.check(G.L().lcu_embed(out_d.ptr, G.dev_keep(bad).ptr, 2, dim, G.dev_keep(table).ptr, vocab, None))
    assert (G.host(out_d, (2, dim)) == 0).all()
    G.B.check(G.L().lcu_embed_u8(out_d.ptr, G.dev_keep(bad).ptr, 2, dim, G.dev_keep(codes).ptr,
                                 G.dev_keep(scales).ptr, 128, vocab, None))
    assert (G.host(out_d, (2, dim)) == 0).all()
    G.release()
    # uint8 rows of more than one piece of 4096 codes (sixteen codes per thread), and a block size that is
    # not a multiple of 16 (one code per thread)
    for vocab, dim, block in ((40, 6656, 128), (40, 4096 + 16, 16), (50, 480, 24)):
        table = normal((vocab, dim), 0, 901, 0.02)
        codes, scales = O.quantize_absmax_u8(table, block)
        ids = np.array([vocab - 1, 0, 7, vocab, 7], dtype=np.int16)
        out_d = G.empty((len(ids), dim))
        G.B.check(G.L().lcu_embed_u8(out_d.ptr, G.dev_keep(ids).ptr, len(ids), dim, G.dev_keep(codes).ptr,
                                     G.dev_keep(scales).ptr, block, vocab, None))
        got = G.host(out_d, (len(ids), dim))
        want = O.embed_u8(np.where(ids < vocab, ids, 0).astype(np.int16), codes, scales, block)
        want[3] = 0
        assert (got.view(np.uint16) == want.view(np.uint16)).all()
        G.release()


def test_embed_rmsnorm_equals_embed_then_rmsnorm(gpu):
    """The one-token step's first launch: the gathered row and its norm, to the bit what lcu_embed[_u8] and
    lcu_rmsnorm give one after the other (and so what the oracle gives for them)."""
    G = gpu
    for vocab, dim, block in ((300, 4096, 0), (300, 4096, 128), (100, 6656, 128), (64, 264, 0), (64, 264, 8), (20, 8192, 64)):
        table = normal((vocab, dim), 0, 910, 0.02)
        w = normal((dim,), 0, 911, 1.0)
        ids = np.array([vocab - 1, 0, 5, vocab, -3, 5], dtype=np.int16)
        x_d, n_d = G.empty((len(ids), dim)), G.empty((len(ids), dim))
        safe = np.where((ids >= 0) & (ids < vocab), ids, 0).astype(np.int16)
        if block:
            codes, scales = O.quantize_absmax_u8(table, block)
            G.B.check(G.L().lcu_embed_rmsnorm(x_d.ptr, n_d.ptr, G.dev_keep(ids).ptr, len(ids), dim, G.dev_keep(codes).ptr,
                                              G.dev_keep(scales).ptr, block, vocab, G.dev_keep(w).ptr, 1e-6, None))
            rows = O.embed_u8(safe, codes, scales, block)
        else:
            G.B.check(G.L().lcu_embed_rmsnorm(x_d.ptr, n_d.ptr, G.dev_keep(ids).ptr, len(ids), dim, G.dev_keep(table).ptr,
                                              None, 0, vocab, G.dev_keep(w).ptr, 1e-6, None))
            rows = O.embed(safe, table)
        rows[3] = 0
        rows[4] = 0
        assert (G.host(x_d, (len(ids), dim)).view(np.uint16) == rows.view(np.uint16)).all()
        assert (G.host(n_d, (len(ids), dim)).view(np.uint16) == O.rms_norm(rows, w, 1e-6).view(np.uint16)).all()
        G.release()
    out = G.empty((1, 8200))
    assert G.L().lcu_embed_rmsnorm(out.ptr, out.ptr, out.ptr, 1, 8200, out.ptr, None, 0, 10, out.ptr, 1e-6, None) != 0
    G.release()


def test_argmax_first_maximum(gpu):
    G = gpu
    out_d = G.empty((1,), np.int32)
    rng = np.random.default_rng(0)
    for n in (5, 1024, 32000, 40001):
        p = rng.random(n).astype(np.float16)
        m = p.max()
        ties = rng.choice(n, size=min(4, n), replace=False)
        p[ties] = m
        G.B.check(G.L().lcu_argmax_f16(out_d.ptr, G.dev_keep(p).ptr, n, None))
        expected = int(np.flatnonzero(p == m)[0])
        assert int(G.host(out_d, (1,), np.int32)[0]) == O.argmax_first(p) == expected
    G.release()


def test_error_stats(gpu):
    G = gpu
    for n in (1, 255, 4096, 1 << 20, (1 << 22) + 77):
        a = normal((n,), 8, 1, 1.0)
        b = normal((n,), 8, 2, 1.0)
        out = G.empty((3,), np.float32)
        da, db = G.dev_keep(a), G.dev_keep(b)
        G.B.check(G.L().lcu_error_stats(out.ptr, da.ptr, db.ptr, n, None))
        got = G.host(out, (3,), np.float32)
        want = O.error_stats(a, b)
        assert got[1] == want[1]                                  # the largest difference is exact
        assert np.allclose(got[[0, 2]], want[[0, 2]], rtol=1e-5)  # fp32 partial sums against double
        # run to run identical (the reference's atomics are not)
        G.B.check(G.L().lcu_error_stats(out.ptr, da.ptr, db.ptr, n, None))
        assert (G.host(out, (3,), np.float32) == got).all()
        G.B.check(G.L().lcu_error_stats(out.ptr, da.ptr, da.ptr, n, None))
        assert (G.host(out, (3,), np.float32) == 0).all()
        G.release()


def test_memset_and_copies(gpu):
    G = gpu
    for n in (1, 15, 16, 17, 4099, 1 << 20):
        buf = G.empty((n + 32,), np.uint8)
        G.B.check(G.L().lcu_memset(buf.ptr, 0xAB, n + 32, None))
        G.B.check(G.L().lcu_memset(buf.ptr + 3, 0x11, n, None))
        h = G.host(buf, (n + 32,), np.uint8)
        assert (h[:3] == 0xAB).all() and (h[3:3 + n] == 0x11).all() and (h[3 + n:] == 0xAB).all()


ATT_CASES = [(1, 1), (1, 2), (1, 255), (1, 256), (1, 257), (1, 577), (1, 2048), (5, 5), (64, 64), (70, 70),
             (512, 512), (3, 130), (40, 300), (300, 2100), (64, 4096), (1, 4096)]


@pytest.mark.parametrize("n,T", ATT_CASES)
def test_attention(gpu, n, T):
    G = gpu
    heads, dim = 4, 512
    start = T - n
    q = normal((n, dim), 0, 1000, 1.0)
    k = normal((T, dim), 0, 1001, 1.0)
    v = normal((T, dim), 0, 1002, 1.0)
    out_d = G.empty((n, dim))
    G.B.check(G.L().lcu_attention(out_d.ptr, G.dev_keep(q).ptr, G.dev_keep(k).ptr, G.dev_keep(v).ptr, n, T, start, dim,
                                  heads, None))
    got = G.host(out_d, (n, dim))
    ref = O.attention(q, k, v, heads, start)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05  # fp32 summation order only
    if start == 0:
        assert G.ulp_mismatch(got[0], v[0]) == 0.0  # causal row 0 sees only itself
    # the oracle restates the kernels' own sums (for several rows: the matrix cores' steps), every bit
    if n == 1:
        assert G.ulp_mismatch(got, O.attention_decode_kernel_order(q, k, v, heads)) == 0.0
    else:
        assert G.ulp_mismatch(got, O.attention_prefill_kernel_order(q, k, v, heads, start)) == 0.0
    G.release()


@pytest.mark.parametrize("n,T", [(512, 512), (1, 577), (1, 2048), (64, 1024), (512, 2048), (33, 1100)])
def test_attention_llama7b_heads(gpu, n, T):
    """32 heads at dim 4096, the shapes of the benchmark configurations."""
    G = gpu
    heads, dim = 32, 4096
    start = T - n
    q = normal((n, dim), 0, 1010, 1.0)
    k = normal((T, dim), 0, 1011, 1.0)
    v = normal((T, dim), 0, 1012, 1.0)
    out_d = G.empty((n, dim))
    G.B.check(G.L().lcu_attention(out_d.ptr, G.dev_keep(q).ptr, G.dev_keep(k).ptr, G.dev_keep(v).ptr, n, T, start, dim,
                                  heads, None))
    got = G.host(out_d, (n, dim))
    ref = O.attention(q, k, v, heads, start)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.05
    if n == 1:
        assert G.ulp_mismatch(got, O.attention_decode_kernel_order(q, k, v, heads)) == 0.0
    else:
        assert G.ulp_mismatch(got, O.attention_prefill_kernel_order(q, k, v, heads, start)) == 0.0
    G.release()


def test_attention_decode_twice_reuses_workspace(gpu):
    # the split-T decode path keeps arrival counters in a workspace; back-to-back calls must agree
    G = gpu
    heads, dim, T = 32, 4096, 2048
    q = normal((1, dim), 0, 1100, 1.0)
    k = normal((T, dim), 0, 1101, 1.0)
    v = normal((T, dim), 0, 1102, 1.0)
    kd, vd, qd = G.dev_keep(k), G.dev_keep(v), G.dev_keep(q)
    ref = O.attention(q, k, v, heads, T - 1)
    out_d = G.empty((1, dim))
    for T_use in (T, 700, T):
        G.B.check(G.L().lcu_attention(out_d.ptr, qd.ptr, kd.ptr, vd.ptr, 1, T_use, T_use - 1, dim, heads, None))
        got = G.host(out_d, (1, dim))
        want = ref if T_use == T else O.attention(q, k[:T_use], v[:T_use], heads, T_use - 1)
        assert G.max_abs_rel(got, want) <= TOL
    assert G.L().lcu_attention(out_d.ptr, qd.ptr, kd.ptr, vd.ptr, 1, 10, 5, dim, heads, None) == -2
    assert G.L().lcu_attention(out_d.ptr, qd.ptr, kd.ptr, vd.ptr, 1, 10, 9, dim, 31, None) == -2
    G.release()


@pytest.mark.parametrize("heads,ctx", [(32, 1024), (52, 2048), (3, 4096)])
def test_attention_decode_spread_in_a_replayed_graph(gpu, heads, ctx):
    """lcu_attention_decode_spread (eight workgroups per head that hand their scores over inside the launch):
    two calls with different salts captured in one graph, replayed with the position and the step counter
    changed on the device between replays (positions going up and down, so rows hold scores of earlier
    epochs), every replay bit-exact against the kernel-order oracle and against lcu_attention_decode; no
    bounded wait ran out."""
    import ctypes as C
    G = gpu
    L = G.L()
    dim = heads * 128
    k = [normal((ctx, dim), 0, 1200 + i, 1.0) for i in range(2)]
    v = [normal((ctx, dim), 0, 1210 + i, 1.0) for i in range(2)]
    q = [normal((1, dim), 0, 1220 + i, 1.0) for i in range(2)]
    kd, vd, qd = [G.dev_keep(a) for a in k], [G.dev_keep(a) for a in v], [G.dev_keep(a) for a in q]
    out = [G.empty((1, dim)) for _ in range(2)]
    old = G.empty((1, dim))
    stream = C.c_void_p()
    G.B.check(L.lcu_stream_create(C.byref(stream)))
    state = G.B.DeviceBuffer(8)  # int32 position, uint32 step counter
    def set_state(pos, seq):
        a = np.array([pos, seq], dtype=np.uint32)
        G.B.check(L.lcu_h2d(state.ptr, a.ctypes.data_as(C.c_void_p), 8, stream))
        G.B.check(L.lcu_sync(stream))
    def enqueue():
        for i in range(2):
            G.B.check(L.lcu_attention_decode_spread(out[i].ptr, qd[i].ptr, kd[i].ptr, vd[i].ptr, state.ptr, state.ptr + 4,
                                                    i, ctx, dim, heads, stream))
    positions = [5, ctx - 1, 300, 0, 1023 if ctx > 1023 else ctx // 2, 17, ctx - 2]
    set_state(positions[0], 1)
    enqueue()  # eager
    G.B.check(L.lcu_sync(stream))
    G.B.check(L.lcu_graph_begin_capture(stream))
    enqueue()
    graph = C.c_void_p()
    G.B.check(L.lcu_graph_end_capture(stream, C.byref(graph)))
    for step, pos in enumerate(positions):
        set_state(pos, 2 + step)
        G.B.check(L.lcu_graph_launch(graph, stream))
        G.B.check(L.lcu_sync(stream))
        T = pos + 1
        for i in range(2):
            got = G.host(out[i], (1, dim))
            assert G.ulp_mismatch(got, O.attention_decode_kernel_order(q[i], k[i][:T], v[i][:T], heads)) == 0.0, (pos, i)
            G.B.check(L.lcu_attention_decode(old.ptr, qd[i].ptr, kd[i].ptr, vd[i].ptr, state.ptr, ctx, dim, heads, stream))
            G.B.check(L.lcu_sync(stream))
            assert G.ulp_mismatch(got, G.host(old, (1, dim))) == 0.0, (pos, i)
    # a step counter that has come round to the same low 21 bits: the caller clears the hand-over words first
    G.B.check(L.lcu_sync_reset(stream))
    set_state(300, 2 + (1 << 21))
    G.B.check(L.lcu_graph_launch(graph, stream))
    G.B.check(L.lcu_sync(stream))
    for i in range(2):
        assert G.ulp_mismatch(G.host(out[i], (1, dim)), O.attention_decode_kernel_order(q[i], k[i][:301], v[i][:301], heads)) == 0.0
    G.B.check(L.lcu_graph_begin_capture(stream))
    assert L.lcu_sync_reset(stream) == -2  # a memset node is not what a captured step may hold
    enqueue()
    graph2 = C.c_void_p()
    G.B.check(L.lcu_graph_end_capture(stream, C.byref(graph2)))
    G.B.check(L.lcu_graph_destroy(graph2))
    count = C.c_uint(123)
    G.B.check(L.lcu_sync_timeouts(stream, C.byref(count)))
    assert count.value == 0
    assert L.lcu_attention_decode_spread(out[0].ptr, qd[0].ptr, kd[0].ptr, vd[0].ptr, state.ptr, state.ptr + 4, 1024, ctx,
                                         dim, heads, stream) == -2
    assert L.lcu_attention_decode_spread(out[0].ptr, qd[0].ptr, kd[0].ptr, vd[0].ptr, state.ptr, None, 0, ctx, dim, heads,
                                         stream) == -2
    G.B.check(L.lcu_graph_destroy(graph))
    G.B.check(L.lcu_stream_destroy(stream))
    state.free()
    G.release()


@pytest.mark.parametrize("heads,ctx", [(32, 1024), (8, 640), (3, 1024), (24, 300)])
def test_decode_attention_wo_norm_equals_its_separate_operators(gpu, heads, ctx):
    """lcu_decode_attention_wo_norm (attention, x += att . Wo^T and the RMS norm behind it in one launch with
    in-launch hand-overs) against lcu_attention_decode + lcu_gemm_f16_nt (beta 1) + lcu_rmsnorm and against the
    kernel-order oracle, bit for bit: eager, captured and replayed with positions going up and down."""
    import ctypes as C
    G = gpu
    L = G.L()
    dim = heads * 128
    eps = 1e-5
    k, v = normal((ctx, dim), 0, 1300, 1.0), normal((ctx, dim), 0, 1301, 1.0)
    q, x0 = normal((1, dim), 0, 1302, 1.0), normal((1, dim), 0, 1303, 1.0)
    wo, nw = normal((dim, dim), 0, 1304, 0.02), normal((dim,), 1, 1305, 0.1)
    kd, vd, qd, wod, nwd = [G.dev_keep(a) for a in (k, v, q, wo, nw)]
    x_f, n_f = G.empty((1, dim)), G.empty((1, dim))       # fused
    x_s, n_s, att_s = G.empty((1, dim)), G.empty((1, dim)), G.empty((1, dim))  # separate
    stream = C.c_void_p()
    G.B.check(L.lcu_stream_create(C.byref(stream)))
    state = G.B.DeviceBuffer(8)
    def set_state(pos, seq):
        a = np.array([pos, seq], dtype=np.uint32)
        G.B.check(L.lcu_h2d(state.ptr, a.ctypes.data_as(C.c_void_p), 8, stream))
        for dst in (x_f, x_s):
            G.B.check(L.lcu_h2d(dst.ptr, x0.ctypes.data_as(C.c_void_p), x0.nbytes, stream))
        G.B.check(L.lcu_sync(stream))
    def fused():
        G.B.check(L.lcu_decode_attention_wo_norm(x_f.ptr, n_f.ptr, qd.ptr, kd.ptr, vd.ptr, wod.ptr, nwd.ptr, eps, state.ptr,
                                                 state.ptr + 4, 7, ctx, dim, heads, stream))
    def check(pos):
        G.B.check(L.lcu_attention_decode(att_s.ptr, qd.ptr, kd.ptr, vd.ptr, state.ptr, ctx, dim, heads, stream))
        G.B.check(L.lcu_gemm_f16_nt(x_s.ptr, att_s.ptr, wod.ptr, 1, dim, dim, 1.0, stream))
        G.B.check(L.lcu_rmsnorm(n_s.ptr, x_s.ptr, nwd.ptr, 1, dim, eps, stream))
        G.B.check(L.lcu_sync(stream))
        got_x, got_n = G.host(x_f, (1, dim)), G.host(n_f, (1, dim))
        assert G.ulp_mismatch(got_x, G.host(x_s, (1, dim))) == 0.0, pos
        assert G.ulp_mismatch(got_n, G.host(n_s, (1, dim))) == 0.0, pos
        T = pos + 1
        att = O.attention_decode_kernel_order(q, k[:T], v[:T], heads)
        want_x = O.matmul_nt(att, wo, flavour=2, beta=1.0, out=x0)
        assert G.ulp_mismatch(got_x, want_x) == 0.0, pos
        assert G.ulp_mismatch(got_n, O.rms_norm(want_x, nw, eps)) == 0.0, pos
    positions = [4, ctx - 1, 200, 0, ctx // 2, ctx - 2]
    set_state(positions[0], 1)
    fused()
    check(positions[0])
    set_state(positions[0], 2)
    G.B.check(L.lcu_graph_begin_capture(stream))
    fused()
    graph = C.c_void_p()
    G.B.check(L.lcu_graph_end_capture(stream, C.byref(graph)))
    for step, pos in enumerate(positions):
        set_state(pos, 3 + step)
        G.B.check(L.lcu_graph_launch(graph, stream))
        check(pos)
    count = C.c_uint(123)
    G.B.check(L.lcu_sync_timeouts(stream, C.byref(count)))
    assert count.value == 0
    assert L.lcu_decode_attention_wo_norm(x_f.ptr, n_f.ptr, qd.ptr, kd.ptr, vd.ptr, wod.ptr, nwd.ptr, eps, state.ptr,
                                          state.ptr + 4, 7, 1025, dim, heads, stream) == -2
    # more workgroups than compute units could not all be resident while they wait for one another
    assert L.lcu_decode_attention_wo_norm(x_f.ptr, n_f.ptr, qd.ptr, kd.ptr, vd.ptr, wod.ptr, nwd.ptr, eps, state.ptr,
                                          state.ptr + 4, 7, ctx, 52 * 128, 52, stream) == -2
    G.B.check(L.lcu_graph_destroy(graph))
    G.B.check(L.lcu_stream_destroy(stream))
    state.free()
    G.release()


@pytest.mark.parametrize("K,N,u8", [(11008, 4096, False), (17920, 6656, True), (4096, 4096, True), (2816, 1024, False),
                                    (512, 8, False), (1024, 8192, False)])
def test_decode_proj_norm_equals_its_separate_operators(gpu, K, N, u8):
    """lcu_decode_proj_norm (x += lhs . W^T and the RMS norm of the new x in one launch; an extra workgroup waits
    inside the launch for the rows) against lcu_gemm_* (beta 1) + lcu_rmsnorm and the kernel-order oracle, bit for
    bit, eager and replayed from a graph with the step counter changed between replays."""
    import ctypes as C
    G = gpu
    L = G.L()
    eps = 1e-6
    lhs = [normal((1, K), 0, 1400 + i, 1.0) for i in range(3)]
    x0 = normal((1, N), 0, 1410, 1.0)
    w, nw = normal((N, K), 0, 1411, 0.02), normal((N,), 1, 1412, 0.3)
    block = 128 if u8 else 0
    if u8:
        codes, scales = O.quantize_absmax_u8(w, block)
        wd, sd = G.dev_keep(codes), G.dev_keep(scales)
    else:
        wd, sd = G.dev_keep(w), None
    nwd = G.dev_keep(nw)
    lhs_d = G.empty((1, K))
    x_f, n_f, x_s, n_s = G.empty((1, N)), G.empty((1, N)), G.empty((1, N)), G.empty((1, N))
    stream = C.c_void_p()
    G.B.check(L.lcu_stream_create(C.byref(stream)))
    state = G.B.DeviceBuffer(8)
    def prepare(seq, which):
        a = np.array([0, seq], dtype=np.uint32)
        G.B.check(L.lcu_h2d(state.ptr, a.ctypes.data_as(C.c_void_p), 8, stream))
        G.B.check(L.lcu_h2d(lhs_d.ptr, lhs[which].ctypes.data_as(C.c_void_p), lhs[which].nbytes, stream))
        for dst in (x_f, x_s):
            G.B.check(L.lcu_h2d(dst.ptr, x0.ctypes.data_as(C.c_void_p), x0.nbytes, stream))
        G.B.check(L.lcu_sync(stream))
    def fused():
        G.B.check(L.lcu_decode_proj_norm(x_f.ptr, n_f.ptr, lhs_d.ptr, wd.ptr, sd.ptr if u8 else None, block, K, N, nwd.ptr,
                                         eps, state.ptr + 4, 3, stream))
    def check(which):
        if u8:
            G.B.check(L.lcu_gemm_f16u8_nt(x_s.ptr, lhs_d.ptr, wd.ptr, sd.ptr, 1, K, N, block, 1.0, stream))
        else:
            G.B.check(L.lcu_gemm_f16_nt(x_s.ptr, lhs_d.ptr, wd.ptr, 1, K, N, 1.0, stream))
        G.B.check(L.lcu_rmsnorm(n_s.ptr, x_s.ptr, nwd.ptr, 1, N, eps, stream))
        G.B.check(L.lcu_sync(stream))
        got_x, got_n = G.host(x_f, (1, N)), G.host(n_f, (1, N))
        assert G.ulp_mismatch(got_x, G.host(x_s, (1, N))) == 0.0, which
        assert G.ulp_mismatch(got_n, G.host(n_s, (1, N))) == 0.0, which
        if u8:
            want_x = O.matmul_nt_u8(lhs[which], codes, scales, block, beta=1.0, out=x0, flavour=2)
        else:
            want_x = O.matmul_nt(lhs[which], w, flavour=2, beta=1.0, out=x0)
        assert G.ulp_mismatch(got_x, want_x) == 0.0, which
        assert G.ulp_mismatch(got_n, O.rms_norm(want_x, nw, eps)) == 0.0, which
    prepare(1, 0)
    fused()
    check(0)
    prepare(2, 0)
    G.B.check(L.lcu_graph_begin_capture(stream))
    fused()
    graph = C.c_void_p()
    G.B.check(L.lcu_graph_end_capture(stream, C.byref(graph)))
    for step in range(4):
        prepare(3 + step, step % 3)
        G.B.check(L.lcu_graph_launch(graph, stream))
        check(step % 3)
    count = C.c_uint(123)
    G.B.check(L.lcu_sync_timeouts(stream, C.byref(count)))
    assert count.value == 0
    assert L.lcu_decode_proj_norm(x_f.ptr, n_f.ptr, lhs_d.ptr, wd.ptr, sd.ptr if u8 else None, block, K, 8200, nwd.ptr, eps,
                                  state.ptr + 4, 3, stream) == -2
    G.B.check(L.lcu_graph_destroy(graph))
    G.B.check(L.lcu_stream_destroy(stream))
    state.free()
    G.release()


@pytest.mark.parametrize("B,dim,heads,ffn,u8", [(8, 4096, 32, 11008, False), (8, 4096, 32, 11008, True), (33, 1024, 8, 2816, False),
                                                (3, 320, 2, 704, False), (1, 512, 4, 1408, True)])
def test_batch_fused_steps_equal_their_separate_operators(gpu, B, dim, heads, ffn, u8):
    """lcu_batch_qkv / lcu_batch_ffn_up / lcu_batch_proj_norm against the operators they fuse, bit for bit: on
    shapes that take the split-K path (partial sums added up by the fused kernel), on shapes that do not
    (dim 320: ragged K; one row) and with uint8 weights."""
    G = gpu
    L = G.L()
    VP = G.B.vp
    ctx, block = 16, (128 if u8 else 0)
    table = VP()
    G.B.check(L.lcu_rope_table_create(G.B.C.byref(table), ctx, dim // heads, 10000.0))
    pos = np.arange(B, dtype=np.int32) % ctx
    x = normal((B, dim), 0, 1700, 1.0)

    def weights(rows, cols, stream):
        w = normal((rows, cols), 0, stream, 0.02)
        if not u8:
            return G.dev_keep(w), None
        c, sc = O.quantize_absmax_u8(w, 128)
        return G.dev_keep(c), G.dev_keep(sc)

    def arr(items):
        return (VP * len(items))(*[(i.ptr if i is not None else None) for i in items])

    def caches():
        k = [G.dev_keep(np.zeros((ctx, dim), dtype=np.float16)) for _ in range(B)]
        v = [G.dev_keep(np.zeros((ctx, dim), dtype=np.float16)) for _ in range(B)]
        return k, v, G.dev_keep(np.array([d.ptr for d in k], dtype=np.uint64)), G.dev_keep(np.array([d.ptr for d in v], dtype=np.uint64))

    xd, pd = G.dev_keep(x), G.dev_keep(pos)
    # Wq, Wk, Wv + rotary + cache append
    qkv = [weights(dim, dim, 1701 + g) for g in range(3)]
    w_arr, s_arr = arr([w for w, _ in qkv]), arr([sc for _, sc in qkv])
    res = []
    for fused in (True, False):
        kc, vc, kptr, vptr = caches()
        q, kt, vt = G.empty((B, dim)), G.empty((B, dim)), G.empty((B, dim))
        if fused:
            G.B.check(L.lcu_batch_qkv(q.ptr, kt.ptr, vt.ptr, xd.ptr, w_arr, s_arr, block, B, dim, heads, kptr.ptr, vptr.ptr,
                                      pd.ptr, table, ctx, None))
        else:
            outs = arr([q, kt, vt])
            if u8:
                G.B.check(L.lcu_gemm_f16u8_nt_multi(outs, xd.ptr, w_arr, s_arr, 3, B, dim, dim, block, 0.0, None))
            else:
                G.B.check(L.lcu_gemm_f16_nt_multi(outs, xd.ptr, w_arr, 3, B, dim, dim, 0.0, None))
            G.B.check(L.lcu_rope_store_batch(q.ptr, kt.ptr, vt.ptr, kptr.ptr, vptr.ptr, pd.ptr, B, dim, heads, table, ctx, None))
        res.append([G.host(q, (B, dim))] + [G.host(c, (ctx, dim)) for c in kc + vc])
    for a, b in zip(*res):
        assert (a.view(np.uint16) == b.view(np.uint16)).all()
    assert np.abs(res[0][0].astype(np.float32)).max() > 0
    # W1, W3 + SiLU
    up = [weights(ffn, dim, 1710 + g) for g in range(2)]
    w_arr, s_arr = arr([w for w, _ in up]), arr([sc for _, sc in up])
    t1, t3, fused_out, sep_out = G.empty((B, ffn)), G.empty((B, ffn)), G.empty((B, ffn)), G.empty((B, ffn))
    G.B.check(L.lcu_batch_ffn_up(fused_out.ptr, t1.ptr, t3.ptr, xd.ptr, w_arr, s_arr, block, B, dim, ffn, None))
    outs = arr([t1, t3])
    if u8:
        G.B.check(L.lcu_gemm_f16u8_nt_multi(outs, xd.ptr, w_arr, s_arr, 2, B, dim, ffn, block, 0.0, None))
    else:
        G.B.check(L.lcu_gemm_f16_nt_multi(outs, xd.ptr, w_arr, 2, B, dim, ffn, 0.0, None))
    G.B.check(L.lcu_silu_mul(sep_out.ptr, t1.ptr, t3.ptr, B * ffn, None))
    assert (G.host(fused_out, (B, ffn)).view(np.uint16) == G.host(sep_out, (B, ffn)).view(np.uint16)).all()
    # W2 with the residual + the next norm
    h = normal((B, ffn), 0, 1720, 0.5)
    hd = G.dev_keep(h)
    w2, s2 = weights(dim, ffn, 1721)
    nw = G.dev_keep(normal((dim,), 0, 1722, 1.0))
    xa, xb, na, nb = G.dev(x), G.dev(x), G.empty((B, dim)), G.empty((B, dim))
    G.B.check(L.lcu_batch_proj_norm(xa.ptr, na.ptr, hd.ptr, w2.ptr, s2.ptr if s2 else None, block, B, ffn, dim, nw.ptr, 1e-6, None))
    if u8:
        G.B.check(L.lcu_gemm_f16u8_nt(xb.ptr, hd.ptr, w2.ptr, s2.ptr, B, ffn, dim, block, 1.0, None))
    else:
        G.B.check(L.lcu_gemm_f16_nt(xb.ptr, hd.ptr, w2.ptr, B, ffn, dim, 1.0, None))
    G.B.check(L.lcu_rmsnorm(nb.ptr, xb.ptr, nw.ptr, B, dim, 1e-6, None))
    assert (G.host(xa, (B, dim)).view(np.uint16) == G.host(xb, (B, dim)).view(np.uint16)).all()
    assert (G.host(na, (B, dim)).view(np.uint16) == G.host(nb, (B, dim)).view(np.uint16)).all()
    G.release()
    L.lcu_free(table)


@pytest.mark.parametrize("n", [1, 5, 1000, 1024, 32000, 32003])
def test_sample_row(gpu, n):
    # integer arithmetic on both sides: the drawn index must agree exactly
    G = gpu
    rng = np.random.default_rng(n)
    rows = [O.softmax_rows(normal((1, n), 0, 1300 + n, 2.0), 0.8)[0],          # a real distribution
            (rng.random(n) * 0.01).astype(np.float16),                         # does not sum to 1
            np.where(rng.random(n) < 0.9, 0, rng.random(n)).astype(np.float16)]  # mostly zeros
    special = (rng.random(n) * 0.5).astype(np.float16)
    special[::7] = np.float16(-1.0)
    special[::11] = np.float16(np.nan)
    special[n // 2] = np.float16(np.inf)
    rows.append(special)
    rows.append(np.zeros(n, dtype=np.float16))
    randoms = [0, 1, 2**63, 2**64 - 1] + [int(v) for v in rng.integers(0, 2**64, 12, dtype=np.uint64)]
    idx_d = G.empty((1,), np.int32)
    for p in rows:
        pd = G.dev_keep(p)
        for r in randoms:
            G.B.check(G.L().lcu_sample_row(idx_d.ptr, pd.ptr, n, r, None, None))
            assert int(G.host(idx_d, (1,), np.int32)[0]) == O.sample_row(p, r), (n, r)
    # the random bits read from device memory (what a captured launch does)
    r = randoms[-1]
    rd = G.dev_keep(np.array([r], dtype=np.uint64))
    G.B.check(G.L().lcu_sample_row(idx_d.ptr, G.dev_keep(rows[0]).ptr, n, 0, rd.ptr, None))
    assert int(G.host(idx_d, (1,), np.int32)[0]) == O.sample_row(rows[0], r)
    assert G.L().lcu_sample_row(idx_d.ptr, None, n, 0, None, None) == -2
    assert G.L().lcu_sample_row(idx_d.ptr, rd.ptr, 0, 0, None, None) == -2
    G.release()


def test_batch_step_operators(gpu):
    """The per-sequence parts of a batched decode step against their single-sequence forms, bit for bit:
    rotary + cache append with a position per row, attention over each sequence's own caches, softmax +
    argmax per row."""
    G = gpu
    L = G.L()
    dim, heads, ctx, B = 512, 4, 40, 3
    pos = np.array([17, 0, 39], dtype=np.int32)
    table = G.B.vp()
    G.B.check(L.lcu_rope_table_create(G.B.C.byref(table), ctx, dim // heads, 10000.0))
    q, k, v = normal((B, dim), 0, 1500, 1.0), normal((B, dim), 0, 1501, 1.0), normal((B, dim), 0, 1502, 1.0)
    kc = [normal((ctx, dim), 0, 1510 + b, 1.0) for b in range(B)]
    vc = [normal((ctx, dim), 0, 1520 + b, 1.0) for b in range(B)]
    kd, vd = [G.dev_keep(a) for a in kc], [G.dev_keep(a) for a in vc]
    kptr = G.dev_keep(np.array([d.ptr for d in kd], dtype=np.uint64))
    vptr = G.dev_keep(np.array([d.ptr for d in vd], dtype=np.uint64))
    qd, kn, vn, pd = G.dev_keep(q), G.dev_keep(k), G.dev_keep(v), G.dev_keep(pos)
    G.B.check(L.lcu_rope_store_batch(qd.ptr, kn.ptr, vn.ptr, kptr.ptr, vptr.ptr, pd.ptr, B, dim, heads, table, ctx, None))
    out_d = G.empty((B, dim))
    G.B.check(L.lcu_attention_decode_batch(out_d.ptr, qd.ptr, kptr.ptr, vptr.ptr, pd.ptr, B, ctx, dim, heads, None))
    q_rot, out = G.host(qd, (B, dim)), G.host(out_d, (B, dim))
    for b in range(B):
        p = int(pos[b])
        # single-sequence forms: lcu_rope on the row at its position, lcu_attention_decode on the caches
        row = G.empty((1, dim))
        G.B.check(L.lcu_rope(row.ptr, G.dev_keep(q[b:b + 1]).ptr, 1, dim, heads, p, table, ctx, None))
        assert (G.host(row, (1, dim)).view(np.uint16) == q_rot[b].view(np.uint16)).all()
        G.B.check(L.lcu_rope(row.ptr, G.dev_keep(k[b:b + 1]).ptr, 1, dim, heads, p, table, ctx, None))
        k_now, v_now = G.host(kd[b], (ctx, dim)), G.host(vd[b], (ctx, dim))
        assert (k_now[p].view(np.uint16) == G.host(row, (1, dim))[0].view(np.uint16)).all()
        assert (v_now[p].view(np.uint16) == v[b].view(np.uint16)).all()
        others = np.arange(ctx) != p
        assert (k_now[others].view(np.uint16) == kc[b][others].view(np.uint16)).all()
        one = G.empty((1, dim))
        G.B.check(L.lcu_attention_decode(one.ptr, G.dev_keep(q_rot[b:b + 1]).ptr, kd[b].ptr, vd[b].ptr,
                                         G.dev_keep(pos[b:b + 1]).ptr, ctx, dim, heads, None))
        assert (G.host(one, (1, dim))[0].view(np.uint16) == out[b].view(np.uint16)).all()
        # and the oracle on the same caches
        ref = O.attention(q_rot[b:b + 1], k_now[:p + 1], v_now[:p + 1], heads, p)
        assert G.max_abs_rel(out[b:b + 1], ref) <= TOL
    n = 1024
    x = normal((B, n), 0, 1530, 1.5)
    probs_d, idx_d = G.empty((B, n)), G.empty((B,), np.int32)
    G.B.check(L.lcu_softmax_argmax_rows(probs_d.ptr, idx_d.ptr, G.dev_keep(x).ptr, B, n, 0.8, None))
    probs, idx = G.host(probs_d, (B, n)), G.host(idx_d, (B,), np.int32)
    p1, i1 = G.empty((n,)), G.empty((1,), np.int32)
    for b in range(B):
        G.B.check(L.lcu_softmax_argmax(p1.ptr, i1.ptr, G.dev_keep(x[b:b + 1]).ptr, n, 0.8, None))
        assert (G.host(p1, (n,)).view(np.uint16) == probs[b].view(np.uint16)).all()
        assert int(G.host(i1, (1,), np.int32)[0]) == int(idx[b]) == O.argmax_first(probs[b])
    assert L.lcu_softmax_argmax_rows(probs_d.ptr, idx_d.ptr, G.dev_keep(x).ptr, B, 1001, 0.8, None) == -2
    assert L.lcu_attention_decode_batch(out_d.ptr, qd.ptr, kptr.ptr, vptr.ptr, pd.ptr, B, ctx, dim, 3, None) == -2
    G.release()


@pytest.mark.parametrize("n,temp", [(32000, 0.8), (32003, 0.9), (5, 1.0), (1024, 0.5)])
def test_softmax_argmax_fused(gpu, n, temp):
    G = gpu
    x = normal((1, n), 0, 1200, 1.3)
    x[0, n // 3] = x.max()  # two equal largest logits: the first index must win
    x[0, n // 3 * 2] = x.max()
    probs_d, idx_d = G.empty((n,)), G.empty((1,), np.int32)
    G.B.check(G.L().lcu_softmax_argmax(probs_d.ptr, idx_d.ptr, G.dev_keep(x).ptr, n, temp, None))
    got = G.host(probs_d, (1, n))
    ref = O.softmax_rows(x, temp)
    assert G.max_abs_rel(got, ref) <= TOL
    assert G.ulp_mismatch(got, ref) < 0.02
    if n % 8 == 0:  # the kernel's own association of the exponential sum, restated: every bit
        assert G.ulp_mismatch(got, O.softmax_logits_kernel_order(x[0], temp)) == 0.0
    assert int(G.host(idx_d, (1,), np.int32)[0]) == O.argmax_first(got) == int(np.flatnonzero(got[0] == got.max())[0])
    assert G.L().lcu_softmax_argmax(probs_d.ptr, idx_d.ptr, probs_d.ptr, n, temp, None) == -2
    G.release()
