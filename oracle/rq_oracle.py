"""ctypes loader for the CPU oracle (librq_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the benchmark's cpu_baseline leg.
The shipped package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librq_oracle.so")

TYPE_W4A4 = 44
TYPE_W4A4H = 45
BLOCK_BYTES = 144
BLOCK_CODES = 256

BLOCK_DTYPE = np.dtype([("d", "<f4"), ("sum", "<i4"), ("pad", "<i4", (2,)), ("qs", "<u4", (32,))])
assert BLOCK_DTYPE.itemsize == BLOCK_BYTES


def build():
    """Compile the oracle with its Makefile (gcc only)."""
    subprocess.run(["make", "-C", _HERE, "-B", "librq_oracle.so"], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c_f32p = ctypes.POINTER(ctypes.c_float)
        L.rqo_hadamard_factor.argtypes = [ctypes.c_int64, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.rqo_hadamard_factor.restype = ctypes.c_int
        L.rqo_paley.argtypes = [ctypes.c_int, ctypes.c_void_p]
        L.rqo_hadamard.argtypes = [c_f32p, ctypes.c_int64, ctypes.c_int]
        L.rqo_resolve_clip.argtypes = [ctypes.c_float, ctypes.c_float]
        L.rqo_resolve_clip.restype = ctypes.c_float
        L.rqo_env_clip.argtypes = [ctypes.c_int]
        L.rqo_env_clip.restype = ctypes.c_float
        L.rqo_tensor_clip.argtypes = [ctypes.c_void_p]
        L.rqo_tensor_clip.restype = ctypes.c_float
        L.rqo_rot_check.argtypes = [ctypes.c_int32, ctypes.c_int64]
        L.rqo_rot_check.restype = ctypes.c_int64
        L.rqo_quantize_row_a.argtypes = [c_f32p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int]
        L.rqo_quantize_row_a4h.argtypes = [c_f32p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float,
                                           ctypes.c_int64, ctypes.c_int]
        L.rqo_vec_dot.argtypes = [ctypes.c_int64, c_f32p, ctypes.c_void_p, ctypes.c_void_p]
        L.rqo_quantize_row_w.argtypes = [c_f32p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int]
        L.rqo_quantize_row_w4a4h.argtypes = [c_f32p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        L.rqo_dequantize_row_w.argtypes = [ctypes.c_void_p, c_f32p, ctypes.c_int64, ctypes.c_int]
        L.rqo_dequantize_row_a.argtypes = [ctypes.c_void_p, c_f32p, ctypes.c_int64, ctypes.c_int]
        L.rqo_mul_mat.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, c_f32p,
                                  ctypes.c_int64, ctypes.c_int64, c_f32p, ctypes.c_int64, ctypes.c_float,
                                  ctypes.c_int64, ctypes.c_int, ctypes.c_int]
        L.rqo_mul_mat.restype = ctypes.c_int
        _lib = L
    return _lib


def _f32p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def hadamard_factor(n):
    p, m = ctypes.c_int(0), ctypes.c_int(0)
    ok = lib().rqo_hadamard_factor(n, ctypes.byref(p), ctypes.byref(m))
    return (p.value, m.value) if ok else None


def paley(p):
    A = np.zeros((p, p), dtype=np.int8)
    lib().rqo_paley(p, A.ctypes.data)
    return A


def hadamard(x, transpose=False):
    """Returns x H (a new float32 array); x is one rotation block."""
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    lib().rqo_hadamard(_f32p(y), y.size, int(transpose))
    return y


def quantize_row_a(x, clip=1.0, G=64):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(x.size // BLOCK_CODES, dtype=BLOCK_DTYPE)
    lib().rqo_quantize_row_a(_f32p(x), y.ctypes.data, x.size, clip, G)
    return y


def quantize_row_a4h(x, clip=1.0, n_rot=None, G=64):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(x.size // BLOCK_CODES, dtype=BLOCK_DTYPE)
    lib().rqo_quantize_row_a4h(_f32p(x), y.ctypes.data, x.size, clip, n_rot or x.size, G)
    return y


def vec_dot(w_row, a_row):
    out = np.zeros(1, dtype=np.float32)
    lib().rqo_vec_dot(w_row.size * BLOCK_CODES, _f32p(out), w_row.ctypes.data, a_row.ctypes.data)
    return out[0]


def quantize_rows_w(w, hadamard=False, n_rot=None, wgroup=0):
    """w: [N, K] float32 -> [N, K/256] blocks, with the reference's weight-side quantizer."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    y = np.zeros((N, K // BLOCK_CODES), dtype=BLOCK_DTYPE)
    for r in range(N):
        if hadamard:
            lib().rqo_quantize_row_w4a4h(_f32p(w[r]), y[r].ctypes.data, K, n_rot or K, wgroup)
        else:
            lib().rqo_quantize_row_w(_f32p(w[r]), y[r].ctypes.data, K, wgroup)
    return y


def dequantize_row_w(blocks, hadamard=False):
    y = np.zeros(blocks.size * BLOCK_CODES, dtype=np.float32)
    lib().rqo_dequantize_row_w(blocks.ctypes.data, _f32p(y), y.size, int(hadamard))
    return y


def dequantize_row_a(blocks, hadamard=False):
    y = np.zeros(blocks.size * BLOCK_CODES, dtype=np.float32)
    lib().rqo_dequantize_row_a(blocks.ctypes.data, _f32p(y), y.size, int(hadamard))
    return y


def mul_mat(type_, w_blocks, x, clip, n_rot=0, G=64, n_threads=None):
    """w_blocks: [N, K/256] blocks; x: [M, K] float32 -> y [M, N] float32 (the reference CPU MUL_MAT)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w_blocks = np.ascontiguousarray(w_blocks)
    N, nb = w_blocks.shape
    K = nb * BLOCK_CODES
    M = x.shape[0]
    assert x.shape[1] == K
    y = np.zeros((M, N), dtype=np.float32)
    if n_threads is None:
        n_threads = min(os.cpu_count() or 1, 64)
    rc = lib().rqo_mul_mat(type_, w_blocks.ctypes.data, K, N, _f32p(x), K, M, _f32p(y), N, clip,
                           n_rot, G, n_threads)
    if rc != 0:
        raise ValueError("oracle: impossible shape")
    return y
