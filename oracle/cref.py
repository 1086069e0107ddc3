"""ctypes loader of oracle/libmlp_ref.so (the plain-C checker).  Test infrastructure."""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_DIR, "libmlp_ref.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _DIR, "-s"], check=True)


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            build()
        _lib = ctypes.CDLL(_PATH)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def silu_mul_bf16(gate_u16, up_u16, round_silu=False):
    g = np.ascontiguousarray(gate_u16, dtype=np.uint16)
    u = np.ascontiguousarray(up_u16, dtype=np.uint16)
    out = np.empty_like(g)
    M, D = g.shape
    load().ref_silu_mul_bf16(_p(g), ctypes.c_long(D), _p(u), ctypes.c_long(D), _p(out), ctypes.c_long(D),
                             ctypes.c_long(M), ctypes.c_long(D), ctypes.c_int(int(round_silu)))
    return out


def rmsnorm_bf16(x_u16, w_u16, eps):
    x = np.ascontiguousarray(x_u16, dtype=np.uint16)
    w = np.ascontiguousarray(w_u16, dtype=np.uint16)
    out = np.empty_like(x)
    M, H = x.shape
    load().ref_rmsnorm_bf16(_p(x), _p(w), _p(out), ctypes.c_long(M), ctypes.c_long(H), ctypes.c_float(eps))
    return out


def gemm_nt_f32(a, w):
    a = np.ascontiguousarray(a, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    M, K = a.shape
    N = w.shape[0]
    c = np.empty((M, N), dtype=np.float32)
    load().ref_gemm_nt_f32(_p(a), _p(w), _p(c), ctypes.c_long(M), ctypes.c_long(N), ctypes.c_long(K))
    return c


def gemm_nt_bf16(a_u16, w_u16):
    a = np.ascontiguousarray(a_u16, dtype=np.uint16)
    w = np.ascontiguousarray(w_u16, dtype=np.uint16)
    M, K = a.shape
    N = w.shape[0]
    c = np.empty((M, N), dtype=np.uint16)
    load().ref_gemm_nt_bf16(_p(a), _p(w), _p(c), ctypes.c_long(M), ctypes.c_long(N), ctypes.c_long(K))
    return c
