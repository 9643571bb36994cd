"""ctypes front end of ``int4_oracle.c`` (test infrastructure only).

The shared object is built by ``make -C oracle`` (or ``__graft_entry__.build``);
loading never compiles anything.
"""

from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libint4_oracle.so")

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is not built: run `make -C oracle`")
        lib = ctypes.CDLL(LIB_PATH)
        lib.vrl_oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.vrl_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        lib.vrl_oracle_bf16_to_f32.restype = ctypes.c_float
        lib.vrl_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib = lib
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _prep(qweight, scales_bits, qzeros):
    return (np.ascontiguousarray(qweight, dtype=np.int32),
            np.ascontiguousarray(scales_bits, dtype=np.uint16),
            np.ascontiguousarray(qzeros, dtype=np.int32))


def _ok(rc):
    if rc != 0:
        raise ValueError("oracle rejected the shapes")


def f32_to_bf16_bits(values):
    lib = load()
    v = np.asarray(values, dtype=np.float32)
    out = np.fromiter((lib.vrl_oracle_f32_to_bf16(float(t)) for t in v.ravel()),
                      dtype=np.uint16, count=v.size)
    return out.reshape(v.shape)


def dequant_bf16(qweight, scales_bits, qzeros, group_size):
    lib = load()
    qw, sc, qz = _prep(qweight, scales_bits, qzeros)
    N, K = qw.shape[0], qw.shape[1] * 8
    w = np.empty((N, K), dtype=np.uint16)
    _ok(lib.vrl_oracle_dequant_bf16(_p(qw), _p(sc), _p(qz), _p(w), N, K, int(group_size)))
    return w


def gemv_f64(x_bits, qweight, scales_bits, qzeros, group_size):
    """Returns (y float64 [M,N], sum|x w| float64 [M,N])."""
    lib = load()
    qw, sc, qz = _prep(qweight, scales_bits, qzeros)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x.shape
    N = qw.shape[0]
    y = np.empty((M, N), dtype=np.float64)
    ya = np.empty((M, N), dtype=np.float64)
    _ok(lib.vrl_oracle_gemv_f64(_p(x), _p(qw), _p(sc), _p(qz), _p(y), _p(ya),
                                M, N, K, int(group_size)))
    return y, ya


def gemv_bf16(x_bits, qweight, scales_bits, qzeros, group_size):
    lib = load()
    qw, sc, qz = _prep(qweight, scales_bits, qzeros)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x.shape
    N = qw.shape[0]
    y = np.empty((M, N), dtype=np.uint16)
    _ok(lib.vrl_oracle_gemv_bf16(_p(x), _p(qw), _p(sc), _p(qz), _p(y), M, N, K, int(group_size)))
    return y


def gate_up_silu_bf16(x_bits, qweight, scales_bits, qzeros, group_size):
    lib = load()
    qw, sc, qz = _prep(qweight, scales_bits, qzeros)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x.shape
    inter = qw.shape[0] // 2
    y = np.empty((M, inter), dtype=np.uint16)
    _ok(lib.vrl_oracle_gate_up_silu_bf16(_p(x), _p(qw), _p(sc), _p(qz), _p(y),
                                         M, inter, K, int(group_size)))
    return y
