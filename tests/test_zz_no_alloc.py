"""lcu_attention_decode_static: attention of one new token without any allocation (its long-row
scores live in a static device array).  Held to lcu_attention, bit for bit, on two calls in a row,
the second with a shorter row, and to its size limits."""
import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import gpu_helpers as G
    G.setup()
    return G


def normal(shape, seed, stream, std):
    n = int(np.prod(shape))
    return O.fill_normal_f16(n, seed, stream, std).reshape(shape)


def test_static_decode_attention_equals_lcu_attention(gpu):
    G = gpu
    L = G.L()
    heads, dim = 32, 4096
    T_max = 2048
    q = normal((1, dim), 0, 2100, 1.0)
    k = normal((T_max, dim), 0, 2101, 1.0)
    v = normal((T_max, dim), 0, 2102, 1.0)
    qd, kd, vd = G.dev_keep(q), G.dev_keep(k), G.dev_keep(v)
    out_a, out_b = G.empty((1, dim)), G.empty((1, dim))
    # two calls in a row on the shared array, the second with a shorter row; then a short row that
    # takes the single-launch form and a long one again
    for T in (2048, 1500, 600, 1025):
        G.B.check(L.lcu_attention_decode_static(out_a.ptr, qd.ptr, kd.ptr, vd.ptr, T, dim, heads, None))
        G.B.check(L.lcu_attention(out_b.ptr, qd.ptr, kd.ptr, vd.ptr, 1, T, T - 1, dim, heads, None))
        a, b = G.host(out_a, (1, dim)), G.host(out_b, (1, dim))
        assert (a.view(np.uint16) == b.view(np.uint16)).all(), T
        assert G.ulp_mismatch(a, O.attention_decode_kernel_order(q, k[:T], v[:T], heads)) == 0.0, T
    # beyond the static array: a clear error, nothing launched
    assert L.lcu_attention_decode_static(out_a.ptr, qd.ptr, kd.ptr, vd.ptr, 4097, dim, heads, None) == -2
    assert b"4096" in L.lcu_last_error()
    assert L.lcu_attention_decode_static(out_a.ptr, qd.ptr, kd.ptr, vd.ptr, 100, 65 * 128, 65, None) == -2
    assert L.lcu_attention_decode_static(out_a.ptr, qd.ptr, kd.ptr, vd.ptr, 0, dim, heads, None) == -2
    G.release()
