"""Shared helpers of the GPU parity tests: device arrays through the C ABI, error metrics."""
import ctypes as C

import numpy as np

import lcu

P = lcu.package()
B = P.binding


def L():
    return P.lib()


def setup():
    B.init(0)


def dev(a):
    return B.to_device(np.ascontiguousarray(a))


def host(buf, shape, dtype=np.float16):
    return B.from_device(buf, shape, dtype)


def empty(shape, dtype=np.float16):
    return B.empty(shape, dtype)


def sync():
    B.check(L().lcu_sync(None), "sync")


def max_abs_rel(a, ref):
    """max |a - ref| / max |ref|: the `max-abs-rel` of the acceptance bar (1e-2 for fp16 outputs)."""
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(a - ref)) / max(np.max(np.abs(ref)), 1e-30))


def ulp_mismatch(a, ref):
    """fraction of fp16 elements whose bit patterns differ"""
    return float((np.asarray(a).view(np.uint16) != np.asarray(ref).view(np.uint16)).mean())


def gemm_f16(x, w, beta=0.0, out=None):
    M, K = x.shape
    N = w.shape[0]
    o = dev(out) if out is not None else dev(np.zeros((M, N), dtype=np.float16))
    B.check(L().lcu_gemm_f16_nt(o.ptr, dev_keep(x).ptr, dev_keep(w).ptr, M, K, N, beta, None), "gemm_f16")
    return host(o, (M, N))


def gemm_u8(x, codes, scales, block, beta=0.0, out=None):
    M, K = x.shape
    N = codes.shape[0]
    o = dev(out) if out is not None else dev(np.zeros((M, N), dtype=np.float16))
    B.check(L().lcu_gemm_f16u8_nt(o.ptr, dev_keep(x).ptr, dev_keep(codes).ptr, dev_keep(scales).ptr, M, K, N, block,
                                  beta, None), "gemm_u8")
    return host(o, (M, N))


_keep = []


def dev_keep(a):
    """device copy kept alive until release() (asynchronous launches read it later)"""
    b = dev(a)
    _keep.append(b)
    return b


def release():
    sync()
    for b in _keep:
        b.free()
    _keep.clear()
