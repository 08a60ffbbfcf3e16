"""ctypes access to oracle/_build/libqmm_ref.so (the C restatement).
TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes as C

import numpy as np

from .build import LIB, build

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not LIB.exists():
            build(verbose=False)
        _lib = C.CDLL(str(LIB))
        _lib.ref_num_threads.restype = C.c_int
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def num_threads() -> int:
    return int(lib().ref_num_threads())


def set_num_threads(n: int) -> None:
    lib().ref_set_num_threads(C.c_int(n))


def unpack_codes(w: np.ndarray, bits: int) -> np.ndarray:
    w = np.ascontiguousarray(w, np.uint32)
    out = np.empty(w.shape[:-1] + (w.shape[-1] * (32 // bits),), np.uint8)
    lib().ref_unpack_codes(_p(w), _p(out), C.c_int64(w.size), C.c_int(bits))
    return out


def dequantize(w, scales, biases, bits: int, two_roundings: bool = True) -> np.ndarray:
    w = np.ascontiguousarray(w, np.uint32)
    s = np.ascontiguousarray(scales, np.uint16)
    b = np.ascontiguousarray(biases, np.uint16)
    K = w.shape[-1] * (32 // bits)
    rows = w.size // w.shape[-1]
    out = np.empty(w.shape[:-1] + (K,), np.uint16)
    lib().ref_dequantize(_p(w), _p(s), _p(b), _p(out), C.c_int64(rows), C.c_int(K), C.c_int(bits),
                         C.c_int(int(two_roundings)))
    return out


def qmm_t(x_bits: np.ndarray, w, scales, biases, bits: int) -> np.ndarray:
    """x bf16 bits [M,K] -> y bf16 bits [M,N]."""
    x = np.ascontiguousarray(x_bits, np.uint16)
    w = np.ascontiguousarray(w, np.uint32)
    s = np.ascontiguousarray(scales, np.uint16)
    b = np.ascontiguousarray(biases, np.uint16)
    M, K = x.shape
    N = w.shape[0]
    assert w.shape[1] * (32 // bits) == K
    y = np.empty((M, N), np.uint16)
    lib().ref_qmm_t(_p(x), _p(w), _p(s), _p(b), _p(y), C.c_int(M), C.c_int(N), C.c_int(K),
                    C.c_int(bits))
    return y
