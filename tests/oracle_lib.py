"""ctypes binding of the CPU oracle (oracle/liboracle.so).  Test infrastructure only.

fp16 arrays are numpy float16; they cross the boundary as their uint16 bit patterns.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_LIB_PATH = os.path.join(ORACLE_DIR, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i, f, u64, sz = C.c_void_p, C.c_int, C.c_float, C.c_uint64, C.c_size_t
        L.orc_fill_normal_f16.argtypes = [vp, sz, u64, u64, f]
        L.orc_quantize_absmax_u8.argtypes = [vp, vp, vp, sz, sz, i]
        L.orc_dequantize_absmax_u8.argtypes = [vp, vp, vp, sz, sz, i]
        L.orc_matmul_nt.argtypes = [vp, vp, vp, i, i, i, f, i]
        L.orc_matmul_nt_u8.argtypes = [vp, vp, vp, vp, i, i, i, i, f, i]
        L.orc_matmul_nt_kernel_order.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, f, i]
        L.orc_matmul_nt_kernel_order.restype = None
        L.orc_gemm_plan.argtypes = [i, i, i, i, i, i]
        L.orc_gemm_plan.restype = i
        L.orc_mfma_f32_f16.argtypes = [vp, vp, vp, vp, sz, i]
        L.orc_mfma_f32_f16.restype = None
        L.orc_rms_norm.argtypes = [vp, vp, vp, i, i, f]
        L.orc_rotary.argtypes = [vp, vp, i, i, i, i, f]
        L.orc_matmul_qk.argtypes = [vp, vp, vp, i, i, i, i, i]
        L.orc_softmax_rows.argtypes = [vp, vp, i, i, f]
        L.orc_matmul_qkv.argtypes = [vp, vp, vp, i, i, i, i]
        L.orc_silu_mul.argtypes = [vp, vp, vp, sz]
        L.orc_exp_f32.argtypes = [vp, vp, sz]
        L.orc_exp_f32.restype = None
        L.orc_dot2_f32_f16.argtypes = [vp, vp, vp, vp, sz]
        L.orc_dot2_f32_f16.restype = None
        L.orc_attention_decode_kernel_order.argtypes = [vp, vp, vp, vp, i, i, i]
        L.orc_attention_decode_kernel_order.restype = None
        L.orc_attention_prefill_kernel_order.argtypes = [vp, vp, vp, vp, i, i, i, i, i]
        L.orc_attention_prefill_kernel_order.restype = None
        L.orc_softmax_logits_kernel_order.argtypes = [vp, vp, i, f]
        L.orc_softmax_logits_kernel_order.restype = None
        L.orc_embed.argtypes = [vp, vp, i, i, vp]
        L.orc_embed_u8.argtypes = [vp, vp, i, i, vp, vp, i]
        L.orc_error_stats.argtypes = [vp, vp, vp, sz]
        L.orc_error_stats.restype = None
        L.orc_argmax_first.argtypes = [vp, i]
        L.orc_argmax_first.restype = i
        L.orc_sample_row.argtypes = [vp, i, u64]
        L.orc_sample_row.restype = i
        L.orc_step_random.argtypes = [u64, u64]
        L.orc_step_random.restype = u64
        L.orc_model_create.argtypes = [i, i, i, i, i, f, i, i, u64, f]
        L.orc_model_create.restype = vp
        L.orc_model_destroy.argtypes = [vp]
        L.orc_model_ffn_dim.argtypes = [vp]
        L.orc_model_ffn_dim.restype = i
        L.orc_model_tensor.argtypes = [vp, u64, C.POINTER(vp)]
        L.orc_model_tensor.restype = vp
        L.orc_context_create.argtypes = [vp, i, f, i, i]
        L.orc_context_create.restype = vp
        L.orc_context_destroy.argtypes = [vp]
        L.orc_context_clear.argtypes = [vp]
        L.orc_context_start_pos.argtypes = [vp]
        L.orc_context_start_pos.restype = i
        L.orc_context_next_token.argtypes = [vp, vp, i, vp, vp, vp]
        L.orc_context_next_token.restype = i
        L.orc_context_kv.argtypes = [vp, i, vp, vp, i]
        L.orc_num_threads.restype = i
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


def fill_normal_f16(n, seed, stream, std):
    out = np.empty(n, dtype=np.float16)
    lib().orc_fill_normal_f16(_p(out), n, seed, stream, std)
    return out


def quantize_absmax_u8(w, block):
    w = _f16(w)
    rows, cols = w.shape
    codes = np.empty((rows, cols), dtype=np.uint8)
    scales = np.empty((rows, cols // block), dtype=np.float16)
    lib().orc_quantize_absmax_u8(_p(codes), _p(scales), _p(w), rows, cols, block)
    return codes, scales


def dequantize_absmax_u8(codes, scales, block):
    codes = np.ascontiguousarray(codes)
    scales = _f16(scales)
    rows, cols = codes.shape
    out = np.empty((rows, cols), dtype=np.float16)
    lib().orc_dequantize_absmax_u8(_p(out), _p(scales), _p(codes), rows, cols, block)
    return out


def matmul_nt(lhs, rhs, beta=0.0, out=None, flavour=1):
    lhs, rhs = _f16(lhs), _f16(rhs)
    M, K = lhs.shape
    N = rhs.shape[0]
    assert rhs.shape[1] == K
    out = np.zeros((M, N), dtype=np.float16) if out is None else _f16(out).copy()
    lib().orc_matmul_nt(_p(out), _p(lhs), _p(rhs), M, K, N, beta, flavour)
    return out


def matmul_nt_u8(lhs, codes, scales, block, beta=0.0, out=None, flavour=1):
    lhs, scales = _f16(lhs), _f16(scales)
    codes = np.ascontiguousarray(codes)
    M, K = lhs.shape
    N = codes.shape[0]
    out = np.zeros((M, N), dtype=np.float16) if out is None else _f16(out).copy()
    lib().orc_matmul_nt_u8(_p(out), _p(lhs), _p(codes), _p(scales), M, K, N, block, beta, flavour)
    return out


def matmul_nt_kernel_order(lhs, rhs=None, codes=None, scales=None, block=0, beta=0.0, out=None, n_mats=1):
    """flavour 2 for a product launched together with n_mats - 1 others of its shape (fp16 weights in
    rhs, or uint8 codes with scales)"""
    lhs = _f16(lhs)
    M, K = lhs.shape
    if codes is None:
        rhs = _f16(rhs)
        N = rhs.shape[0]
        cp, sp, rp = None, None, _p(rhs)
    else:
        codes, scales = np.ascontiguousarray(codes), _f16(scales)
        N = codes.shape[0]
        cp, sp, rp = _p(codes), _p(scales), None
    out = np.zeros((M, N), dtype=np.float16) if out is None else _f16(out).copy()
    lib().orc_matmul_nt_kernel_order(_p(out), _p(lhs), rp, cp, sp, M, K, N, block, beta, n_mats)
    return out


def gemm_plan(M, K, N, u8=False, block=128, n_mats=1):
    """(groups of wavefronts sharing a K stage, K splits) the HIP dispatcher takes for this product"""
    v = lib().orc_gemm_plan(M, K, N, int(u8), block, n_mats)
    return v // 1000, v % 1000


def mfma_f32_f16(a, b, c):
    """a, b: (n, K) fp16 bit patterns, K = 16 or 32 (any multiple of 8); c: (n,) float32 -> the
    accumulator after the matrix instruction (K / 8 steps of eight products)"""
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    c = np.ascontiguousarray(c, dtype=np.float32)
    assert a.shape == b.shape and a.shape[0] == c.size and a.shape[1] % 8 == 0
    out = np.empty_like(c)
    lib().orc_mfma_f32_f16(_p(out), _p(a), _p(b), _p(c), c.size, a.shape[1])
    return out


def rms_norm(x, w, eps):
    x, w = _f16(x), _f16(w)
    rows, cols = x.shape
    out = np.empty_like(x)
    lib().orc_rms_norm(_p(out), _p(x), _p(w), rows, cols, eps)
    return out


def rotary(x, n_heads, pos_offset=0, theta=10000.0):
    x = _f16(x)
    rows, cols = x.shape
    out = np.empty_like(x)
    lib().orc_rotary(_p(out), _p(x), rows, cols, n_heads, pos_offset, theta)
    return out


def matmul_qk(q, k, n_heads, start_pos):
    q, k = _f16(q), _f16(k)
    n_new, dim = q.shape
    T = k.shape[0]
    out = np.empty((n_heads, n_new, T), dtype=np.float16)
    lib().orc_matmul_qk(_p(out), _p(q), _p(k), n_new, T, dim, n_heads, start_pos)
    return out


def softmax_rows(x, temp=1.0):
    x = _f16(x)
    w = x.shape[-1]
    rows = x.size // w
    out = np.empty_like(x)
    lib().orc_softmax_rows(_p(out), _p(x), rows, w, temp)
    return out


def matmul_qkv(p, v, n_heads):
    p, v = _f16(p), _f16(v)
    _, n_new, T = p.shape
    dim = v.shape[1]
    out = np.empty((n_new, dim), dtype=np.float16)
    lib().orc_matmul_qkv(_p(out), _p(p), _p(v), n_new, T, dim, n_heads)
    return out


def attention(q, k, v, n_heads, start_pos):
    """matmul_qk -> softmax_rows -> matmul_qkv, llama_cu.cu:1161-1171."""
    return matmul_qkv(softmax_rows(matmul_qk(q, k, n_heads, start_pos)), v, n_heads)


def dot2_f32_f16(a, b, c):
    """a, b: (n, 2) fp16 bit patterns (uint16), c: (n,) float32 -> what v_dot2_f32_f16 returns"""
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    c = np.ascontiguousarray(c, dtype=np.float32)
    assert a.shape == b.shape == (c.size, 2)
    out = np.empty_like(c)
    lib().orc_dot2_f32_f16(_p(out), _p(a), _p(b), _p(c), c.size)
    return out


def exp_f32(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_exp_f32(_p(out), _p(x), x.size)
    return out


def attention_prefill_kernel_order(q, k, v, n_heads, start_pos=0):
    """n_new > 1 rows of q against T = start_pos + n_new cached rows, sums in the order of the HIP kernel"""
    q, k, v = _f16(q), _f16(k), _f16(v)
    n_new, dim = q.shape
    T = k.shape[0]
    assert T == start_pos + n_new
    out = np.empty((n_new, dim), dtype=np.float16)
    lib().orc_attention_prefill_kernel_order(_p(out), _p(q), _p(k), _p(v), n_new, T, start_pos, dim, n_heads)
    return out


def attention_decode_kernel_order(q, k, v, n_heads):
    """one new token against T cached rows, sums in the order of the HIP kernels"""
    q, k, v = _f16(q), _f16(k), _f16(v)
    T, dim = k.shape
    out = np.empty((1, dim), dtype=np.float16)
    lib().orc_attention_decode_kernel_order(_p(out), _p(q), _p(k), _p(v), T, dim, n_heads)
    return out


def softmax_logits_kernel_order(x, temp):
    x = _f16(x)
    out = np.empty_like(x)
    lib().orc_softmax_logits_kernel_order(_p(out), _p(x), x.size, temp)
    return out


def silu_mul(a, b):
    a, b = _f16(a), _f16(b)
    out = np.empty_like(a)
    lib().orc_silu_mul(_p(out), _p(a), _p(b), a.size)
    return out


def embed(ids, table):
    ids = np.ascontiguousarray(ids, dtype=np.int16)
    table = _f16(table)
    out = np.empty((len(ids), table.shape[1]), dtype=np.float16)
    lib().orc_embed(_p(out), _p(ids), len(ids), table.shape[1], _p(table))
    return out


def embed_u8(ids, codes, scales, block):
    ids = np.ascontiguousarray(ids, dtype=np.int16)
    codes = np.ascontiguousarray(codes)
    scales = _f16(scales)
    out = np.empty((len(ids), codes.shape[1]), dtype=np.float16)
    lib().orc_embed_u8(_p(out), _p(ids), len(ids), codes.shape[1], _p(codes), _p(scales), block)
    return out


def error_stats(a, b):
    a, b = _f16(a), _f16(b)
    out = np.empty(3, dtype=np.float32)
    lib().orc_error_stats(_p(out), _p(a), _p(b), a.size)
    return out


def sample_row(probs, random):
    probs = _f16(probs)
    return lib().orc_sample_row(_p(probs), probs.size, random)


def step_random(seed, step):
    return lib().orc_step_random(seed, step)


def argmax_first(probs):
    probs = _f16(probs)
    return lib().orc_argmax_first(_p(probs), probs.size)


class Model:
    def __init__(self, dim, multiple_of, n_heads, n_layers, n_vocab, norm_eps=1e-6, q_type=0, qblock=128,
                 seed=0, weight_std=0.02):
        self.dim, self.n_heads, self.n_layers, self.n_vocab = dim, n_heads, n_layers, n_vocab
        self.q_type, self.qblock = q_type, qblock
        self.h = lib().orc_model_create(dim, multiple_of, n_heads, n_layers, n_vocab, norm_eps, q_type, qblock,
                                        seed, weight_std)
        self.ffn = lib().orc_model_ffn_dim(self.h)

    def tensor(self, stream, rows, cols):
        sc = C.c_void_p()
        p = lib().orc_model_tensor(self.h, stream, C.byref(sc))
        if self.q_type == 1:
            codes = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), (rows, cols))
            scales = np.ctypeslib.as_array(C.cast(sc, C.POINTER(C.c_uint16)), (rows, cols // self.qblock))
            return codes, scales.view(np.float16)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint16)), (rows, cols)).view(np.float16), None

    def close(self):
        if self.h:
            lib().orc_model_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()


class Context:
    def __init__(self, model, context_len=2048, temperature=0.8, flavour=1, literal_rope=0):
        self.model = model
        self.context_len = context_len
        self.h = lib().orc_context_create(model.h, context_len, temperature, flavour, literal_rope)

    def clear(self):
        lib().orc_context_clear(self.h)

    @property
    def start_pos(self):
        return lib().orc_context_start_pos(self.h)

    def next_token(self, tokens, want=False):
        tokens = np.ascontiguousarray(tokens, dtype=np.int16)
        n = len(tokens)
        m = self.model
        if not want:
            return lib().orc_context_next_token(self.h, _p(tokens), n, None, None, None)
        hidden = np.empty((n, m.dim), dtype=np.float16)
        logits = np.empty(m.n_vocab, dtype=np.float16)
        probs = np.empty(m.n_vocab, dtype=np.float16)
        tok = lib().orc_context_next_token(self.h, _p(tokens), n, _p(hidden), _p(logits), _p(probs))
        return tok, hidden, logits, probs

    def kv(self, layer, T):
        k = np.empty((T, self.model.dim), dtype=np.float16)
        v = np.empty((T, self.model.dim), dtype=np.float16)
        lib().orc_context_kv(self.h, layer, _p(k), _p(v), T)
        return k, v

    def close(self):
        if self.h:
            lib().orc_context_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()
