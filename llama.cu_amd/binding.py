"""ctypes binding of libllama_cu_amd.so (C ABI: include/llama_cu_hip.h, include/llama_cu_c.h)."""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# LLAMA_CU_AMD_LIB names another build of the same library (the diagnostic one of build.py --timeline)
_LIB_PATH = os.environ.get("LLAMA_CU_AMD_LIB") or os.path.join(_PKG, "libllama_cu_amd.so")
_lib = None


class LcuError(RuntimeError):
    pass


class DeviceProps(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("compute_units", C.c_int), ("lds_bytes_per_block", C.c_int),
                ("l2_bytes", C.c_int), ("clock_khz", C.c_int), ("memory_clock_khz", C.c_int),
                ("memory_bus_bits", C.c_int), ("total_memory", C.c_size_t), ("free_memory", C.c_size_t)]


def lib_path():
    return _LIB_PATH


# name -> (restype, argtypes); the single list of every symbol the headers declare
vp, i32, f32, u64, sz, u32, u16 = C.c_void_p, C.c_int, C.c_float, C.c_uint64, C.c_size_t, C.c_uint32, C.c_uint16
SIGNATURES = {
    # llama_cu_hip.h
    "lcu_init": (i32, [i32]),
    "lcu_last_error": (C.c_char_p, []),
    "lcu_device_get_props": (i32, [i32, C.POINTER(DeviceProps)]),
    "lcu_get_device": (i32, [C.POINTER(i32)]),
    "lcu_set_device": (i32, [i32]),
    "lcu_malloc": (i32, [C.POINTER(vp), sz]),
    "lcu_free": (i32, [vp]),
    "lcu_memset": (i32, [vp, i32, sz, vp]),
    "lcu_h2d": (i32, [vp, vp, sz, vp]),
    "lcu_d2h": (i32, [vp, vp, sz, vp]),
    "lcu_d2d": (i32, [vp, vp, sz, vp]),
    "lcu_stream_create": (i32, [C.POINTER(vp)]),
    "lcu_stream_destroy": (i32, [vp]),
    "lcu_sync": (i32, [vp]),
    "lcu_event_create": (i32, [C.POINTER(vp)]),
    "lcu_event_destroy": (i32, [vp]),
    "lcu_event_record": (i32, [vp, vp]),
    "lcu_event_elapsed_ms": (i32, [C.POINTER(f32), vp, vp]),
    "lcu_gemm_f16_nt": (i32, [vp, vp, vp, i32, i32, i32, f32, vp]),
    "lcu_gemm_f16u8_nt": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, f32, vp]),
    "lcu_quantize_absmax_u8": (i32, [vp, vp, vp, sz, sz, i32, vp]),
    "lcu_dequantize_absmax_u8": (i32, [vp, vp, vp, sz, sz, i32, vp]),
    "lcu_rmsnorm": (i32, [vp, vp, vp, i32, i32, f32, vp]),
    "lcu_rope_table_create": (i32, [C.POINTER(vp), i32, i32, f32]),
    "lcu_rope": (i32, [vp, vp, i32, i32, i32, i32, vp, i32, vp]),
    "lcu_rope_pair": (i32, [vp, vp, i32, i32, i32, i32, vp, i32, vp]),
    "lcu_softmax_rows": (i32, [vp, vp, i32, i32, f32, vp]),
    "lcu_silu_mul": (i32, [vp, vp, vp, sz, vp]),
    "lcu_exp_f32": (i32, [vp, vp, sz, vp]),
    "lcu_attention_decode_static": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "lcu_embed": (i32, [vp, vp, i32, i32, vp, i32, vp]),
    "lcu_embed_u8": (i32, [vp, vp, i32, i32, vp, vp, i32, i32, vp]),
    "lcu_embed_rmsnorm": (i32, [vp, vp, vp, i32, i32, vp, vp, i32, i32, vp, f32, vp]),
    "lcu_argmax_f16": (i32, [vp, vp, i32, vp]),
    "lcu_softmax_argmax": (i32, [vp, vp, vp, i32, f32, vp]),
    "lcu_sample_row": (i32, [vp, vp, i32, u64, vp, vp]),
    "lcu_gemm_f16_nt_multi": (i32, [vp, vp, vp, i32, i32, i32, i32, f32, vp]),
    "lcu_gemm_f16u8_nt_multi": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i32, f32, vp]),
    "lcu_rope_store_batch": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, vp]),
    "lcu_attention_decode_batch": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "lcu_softmax_argmax_rows": (i32, [vp, vp, vp, i32, i32, f32, vp]),
    "lcu_batch_qkv": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, vp, vp, vp, i32, vp]),
    "lcu_batch_ffn_up": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "lcu_batch_proj_norm": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, f32, vp]),
    "lcu_attention": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]),
    "lcu_decode_qkv": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, f32, vp, i32, vp]),
    "lcu_attention_decode": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "lcu_attention_decode_spread": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "lcu_sync_timeouts": (i32, [vp, vp]),
    "lcu_sync_add_timeouts": (i32, [vp, u32]),
    "lcu_softmax_argmax_status": (i32, [vp, vp, vp, i32, f32, vp]),
    "lcu_sync_reset": (i32, [vp]),
    "lcu_decode_proj_norm": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, vp, f32, vp, i32, vp]),
    "lcu_decode_attention_wo_norm": (i32, [vp, vp, vp, vp, vp, vp, vp, C.c_float, vp, vp, i32, i32, i32, i32, vp]),
    "lcu_graph_begin_capture": (i32, [vp]),
    "lcu_graph_end_capture": (i32, [vp, C.POINTER(vp)]),
    "lcu_graph_launch": (i32, [vp, vp]),
    "lcu_graph_destroy": (i32, [vp]),
    "lcu_decode_ffn_up": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    "lcu_decode_logits": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    "lcu_fill_normal_f16": (i32, [vp, sz, u64, u64, f32, vp]),
    "lcu_fill_f16": (i32, [vp, sz, u16, vp]),
    "lcu_error_stats": (i32, [vp, vp, vp, sz, vp]),
    # llama_cu_c.h
    "lcu_model_create_synthetic": (vp, [u32, u32, u32, u32, u32, f32, i32, i32, u64, f32]),
    "lcu_model_load": (vp, [C.c_char_p, i32]),
    "lcu_model_destroy": (None, [vp]),
    "lcu_model_ffn_dim": (u32, [vp]),
    "lcu_model_describe": (None, [vp] + [C.POINTER(u32)] * 5 + [C.POINTER(f32), C.POINTER(i32), C.POINTER(i32)]),
    "lcu_model_read_tensor": (i32, [vp, u64, vp, vp]),
    "lcu_model_tensor_ptr": (i32, [vp, u64, C.POINTER(vp), C.POINTER(vp)]),
    "lcu_model_norm_ptr": (vp, [vp, i32]),
    "lcu_context_create": (vp, [vp, i32, f32]),
    "lcu_context_destroy": (None, [vp]),
    "lcu_context_clear_tokens": (None, [vp]),
    "lcu_context_memory_usage": (sz, [vp]),
    "lcu_context_tokens_left": (sz, [vp]),
    "lcu_context_next_token": (i32, [vp, vp, i32]),
    "lcu_context_read_logits": (i32, [vp, vp]),
    "lcu_context_read_probs": (i32, [vp, vp]),
    "lcu_context_read_hidden": (i32, [vp, vp, i32]),
    "lcu_context_read_kv": (i32, [vp, i32, vp, vp, i32]),
    "lcu_context_stream": (vp, [vp]),
    "lcu_context_hand_over_fallbacks": (i32, [vp]),
    "lcu_context_set_sampling": (None, [vp, i32, u64]),
    "lcu_batch_create": (vp, [vp, i32, i32, f32]),
    "lcu_batch_destroy": (None, [vp]),
    "lcu_batch_n_sequences": (i32, [vp]),
    "lcu_batch_memory_usage": (sz, [vp]),
    "lcu_batch_clear_tokens": (i32, [vp, i32]),
    "lcu_batch_tokens_left": (C.c_long, [vp, i32]),
    "lcu_batch_next_token": (i32, [vp, i32, vp, i32]),
    "lcu_batch_next_tokens": (i32, [vp, vp, vp]),
    "lcu_batch_read_logits": (i32, [vp, vp]),
    "lcu_batch_read_probs": (i32, [vp, vp]),
    "lcu_vocab_load": (vp, [C.c_char_p]),
    "lcu_vocab_destroy": (None, [vp]),
    "lcu_vocab_size": (i32, [vp]),
    "lcu_vocab_tokenize": (i32, [vp, C.c_char_p, sz, i32, vp, i32]),
    "lcu_vocab_piece": (vp, [vp, i32, C.POINTER(sz)]),
    "lcu_vocab_score": (f32, [vp, i32]),
}


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise LcuError("%s is missing: build it with `python llama.cu_amd/build.py`" % _LIB_PATH)
        L = C.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise LcuError("%s failed (%d): %s" % (what or "lcu call", rc, lib().lcu_last_error().decode()))


def init(device=0):
    check(lib().lcu_init(device), "lcu_init")


def device_props(device=0):
    p = DeviceProps()
    check(lib().lcu_device_get_props(device, C.byref(p)), "lcu_device_get_props")
    return p


class DeviceBuffer:
    """Owning device allocation (lcu_malloc / lcu_free)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = vp()
        check(lib().lcu_malloc(C.byref(p), max(self.nbytes, 1)), "lcu_malloc")
        self.ptr = p.value

    def free(self):
        if getattr(self, "ptr", None):
            lib().lcu_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device(a, stream=None):
    a = np.ascontiguousarray(a)
    buf = DeviceBuffer(a.nbytes)
    if a.nbytes:
        check(lib().lcu_h2d(buf.ptr, a.ctypes.data_as(vp), a.nbytes, stream), "lcu_h2d")
        check(lib().lcu_sync(stream), "lcu_sync")  # the numpy array may go away
    buf.shape, buf.dtype = a.shape, a.dtype
    return buf


def from_device(buf, shape=None, dtype=None, stream=None):
    shape = buf.shape if shape is None else shape
    dtype = buf.dtype if dtype is None else dtype
    out = np.empty(shape, dtype=dtype)
    if out.nbytes:
        check(lib().lcu_d2h(out.ctypes.data_as(vp), buf.ptr, out.nbytes, stream), "lcu_d2h")
    return out


def empty(shape, dtype):
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    buf = DeviceBuffer(n)
    buf.shape, buf.dtype = tuple(np.atleast_1d(shape)) if np.isscalar(shape) else tuple(shape), np.dtype(dtype)
    return buf


class Model:
    """llama_model (synthetic weights or a model directory in the reference's file format)."""

    def __init__(self, dim=None, multiple_of=None, n_heads=None, n_layers=None, n_vocab=None, norm_eps=1e-6,
                 q_type=0, qblock=128, seed=0, weight_std=0.02, path=None, context_len=2048):
        L = lib()
        if path is not None:
            self.h = L.lcu_model_load(path.encode(), context_len)
        else:
            self.h = L.lcu_model_create_synthetic(dim, multiple_of, n_heads, n_layers, n_vocab, norm_eps, q_type,
                                                  qblock, seed, weight_std)
        if not self.h:
            raise LcuError("model creation failed: %s" % L.lcu_last_error().decode())
        d, m, h, l, v = u32(), u32(), u32(), u32(), u32()
        eps, qt, qb = f32(), i32(), i32()
        L.lcu_model_describe(self.h, C.byref(d), C.byref(m), C.byref(h), C.byref(l), C.byref(v), C.byref(eps),
                             C.byref(qt), C.byref(qb))
        self.dim, self.multiple_of, self.n_heads, self.n_layers, self.n_vocab = d.value, m.value, h.value, l.value, v.value
        self.norm_eps, self.q_type, self.qblock = eps.value, qt.value, (qb.value or qblock)
        self.ffn = L.lcu_model_ffn_dim(self.h)

    def tensor(self, stream_id, rows, cols):
        if self.q_type == 1:
            codes = np.empty((rows, cols), dtype=np.uint8)
            scales = np.empty((rows, cols // self.qblock), dtype=np.float16)
            rc = lib().lcu_model_read_tensor(self.h, stream_id, codes.ctypes.data_as(vp), scales.ctypes.data_as(vp))
            if rc:
                raise LcuError("lcu_model_read_tensor %d" % rc)
            return codes, scales
        w = np.empty((rows, cols), dtype=np.float16)
        rc = lib().lcu_model_read_tensor(self.h, stream_id, w.ctypes.data_as(vp), None)
        if rc:
            raise LcuError("lcu_model_read_tensor %d" % rc)
        return w, None

    def tensor_ptr(self, stream_id):
        d, s = vp(), vp()
        if lib().lcu_model_tensor_ptr(self.h, stream_id, C.byref(d), C.byref(s)):
            raise LcuError("lcu_model_tensor_ptr")
        return d.value, s.value

    def norm_ptr(self, which):
        return lib().lcu_model_norm_ptr(self.h, which)

    def close(self):
        if getattr(self, "h", None):
            lib().lcu_model_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Context:
    """llama_context: create / next_token / clear_tokens / tokens_left / context_memory_usage."""

    def __init__(self, model, context_len=2048, temperature=0.9):
        self.model = model
        self.context_len = context_len
        self.h = lib().lcu_context_create(model.h, context_len, temperature)
        if not self.h:
            raise LcuError("context creation failed")

    def next_token(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int16)
        return lib().lcu_context_next_token(self.h, t.ctypes.data_as(vp), len(t))

    def clear_tokens(self):
        lib().lcu_context_clear_tokens(self.h)

    def sample_with_seed(self, seed):
        """next_token draws from the probabilities from now on (llama_context::sample_with_seed)."""
        lib().lcu_context_set_sampling(self.h, 1, seed)

    def greedy(self):
        lib().lcu_context_set_sampling(self.h, 0, 0)

    def tokens_left(self):
        return lib().lcu_context_tokens_left(self.h)

    def memory_usage(self):
        return lib().lcu_context_memory_usage(self.h)

    @property
    def stream(self):
        return lib().lcu_context_stream(self.h)

    def hand_over_fallbacks(self):
        return lib().lcu_context_hand_over_fallbacks(self.h)

    def logits(self):
        out = np.empty(self.model.n_vocab, dtype=np.float16)
        check(lib().lcu_context_read_logits(self.h, out.ctypes.data_as(vp)), "read_logits")
        return out

    def probs(self):
        out = np.empty(self.model.n_vocab, dtype=np.float16)
        check(lib().lcu_context_read_probs(self.h, out.ctypes.data_as(vp)), "read_probs")
        return out

    def hidden(self, rows):
        out = np.empty((rows, self.model.dim), dtype=np.float16)
        check(lib().lcu_context_read_hidden(self.h, out.ctypes.data_as(vp), rows), "read_hidden")
        return out

    def kv(self, layer, T):
        k = np.empty((T, self.model.dim), dtype=np.float16)
        v = np.empty((T, self.model.dim), dtype=np.float16)
        check(lib().lcu_context_read_kv(self.h, layer, k.ctypes.data_as(vp), v.ctypes.data_as(vp), T), "read_kv")
        return k, v

    def close(self):
        if getattr(self, "h", None):
            lib().lcu_context_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class BatchContext:
    """llama_batch_context: several sequences over one model, one pass over the weights per step."""

    def __init__(self, model, n_sequences, context_len=2048, temperature=0.9):
        self.model = model
        self.n = n_sequences
        self.h = lib().lcu_batch_create(model.h, n_sequences, context_len, temperature)
        if not self.h:
            raise LcuError("batch context creation failed")

    def next_token(self, sequence, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int16)
        return lib().lcu_batch_next_token(self.h, sequence, t.ctypes.data_as(vp), len(t))

    def next_tokens(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int16)
        if len(t) != self.n:
            raise LcuError("one token per sequence")
        out = np.empty(self.n, dtype=np.int16)
        check(lib().lcu_batch_next_tokens(self.h, t.ctypes.data_as(vp), out.ctypes.data_as(vp)), "next_tokens")
        return [int(v) for v in out]

    def clear_tokens(self, sequence):
        check(lib().lcu_batch_clear_tokens(self.h, sequence), "clear_tokens")

    def tokens_left(self, sequence):
        return lib().lcu_batch_tokens_left(self.h, sequence)

    def memory_usage(self):
        return lib().lcu_batch_memory_usage(self.h)

    def logits(self):
        out = np.empty((self.n, self.model.n_vocab), dtype=np.float16)
        check(lib().lcu_batch_read_logits(self.h, out.ctypes.data_as(vp)), "read_logits")
        return out

    def probs(self):
        out = np.empty((self.n, self.model.n_vocab), dtype=np.float16)
        check(lib().lcu_batch_read_probs(self.h, out.ctypes.data_as(vp)), "read_probs")
        return out

    def close(self):
        if self.h:
            lib().lcu_batch_destroy(self.h)
            self.h = None


class Vocabulary:
    """llama_vocabulary over a vocab file in the reference's format (host only, no GPU needed)."""

    def __init__(self, path):
        self.h = lib().lcu_vocab_load(path.encode())
        if not self.h:
            raise LcuError("could not load vocab file %s" % path)

    def __len__(self):
        return lib().lcu_vocab_size(self.h)

    def tokenize(self, text, bos=True):
        data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        cap = 2 * len(data) + 8
        out = (C.c_int16 * cap)()
        n = lib().lcu_vocab_tokenize(self.h, data, len(data), 1 if bos else 0, out, cap)
        if n < 0 or n > cap:
            raise LcuError("lcu_vocab_tokenize returned %d" % n)
        return list(out[:n])

    def piece(self, token_id):
        n = sz()
        ptr = lib().lcu_vocab_piece(self.h, token_id, C.byref(n))
        if not ptr:
            raise IndexError(token_id)
        return C.string_at(ptr, n.value)

    def score(self, token_id):
        return lib().lcu_vocab_score(self.h, token_id)

    def close(self):
        if getattr(self, "h", None):
            lib().lcu_vocab_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
