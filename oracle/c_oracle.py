"""ctypes binding of the plain-C oracle (oracle/vq_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/vq_oracle.c with gcc (seconds)."""
    src = os.path.join(_HERE, "vq_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libvq_oracle.so"])
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.vqo_h2f.restype = ctypes.c_float
        _lib.vqo_h2f.argtypes = [ctypes.c_uint16]
        _lib.vqo_f2h.restype = ctypes.c_uint16
        _lib.vqo_f2h.argtypes = [ctypes.c_float]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16
    return a.view(np.uint16)


def _codes(a):
    a = np.ascontiguousarray(a)
    assert a.dtype in (np.uint8, np.uint16)
    return a, (8 if a.dtype == np.uint8 else 16)


def _cb3(cb):
    cb = np.ascontiguousarray(cb)
    return cb[None] if cb.ndim == 2 else cb


def _check(rc):
    if rc != 0:
        raise ValueError(f"C oracle rejected the arguments (rc={rc})")


def dequant_b(codes, codebook) -> np.ndarray:
    codes, bits = _codes(codes)
    cb = _cb3(codebook)
    G, E, v = cb.shape
    N, J = codes.shape
    out = np.empty((N, J * v), dtype=np.uint16)
    I64, I = ctypes.c_int64, ctypes.c_int
    _check(lib().vqo_dequant_b(_p(codes), I(bits), _p(_u16(cb)), _p(out), I64(N), I64(J * v), I(v), I(E), I(G)))
    return out.view(np.float16)


def dequant_a(w, codebook) -> np.ndarray:
    w = np.ascontiguousarray(w)
    assert w.dtype == np.uint8
    cb = np.ascontiguousarray(codebook)
    K, Nc = w.shape
    _, E, ratio = cb.shape
    out = np.empty((K, Nc * ratio), dtype=np.uint16)
    I64, I = ctypes.c_int64, ctypes.c_int
    _check(lib().vqo_dequant_a(_p(w), _p(_u16(cb)), _p(out), I64(K), I64(Nc), I(E), I(ratio)))
    return out.view(np.float16)


def vq_gemm_b(x, codes, codebook) -> np.ndarray:
    codes, bits = _codes(codes)
    cb = _cb3(codebook)
    G, E, v = cb.shape
    N, J = codes.shape
    x = np.ascontiguousarray(x)
    M, K = x.shape
    assert K == J * v
    y = np.empty((M, N), dtype=np.uint16)
    I64, I = ctypes.c_int64, ctypes.c_int
    _check(lib().vqo_vq_gemm_b(_p(_u16(x)), _p(codes), I(bits), _p(_u16(cb)), _p(y),
                               I64(M), I64(K), I64(N), I(v), I(E), I(G)))
    return y.view(np.float16)


def vq_gemm_a(x, w, codebook) -> np.ndarray:
    w = np.ascontiguousarray(w)
    cb = np.ascontiguousarray(codebook)
    x = np.ascontiguousarray(x)
    M, K = x.shape
    K2, Nc = w.shape
    assert K == K2
    _, E, ratio = cb.shape
    y = np.empty((M, Nc * ratio), dtype=np.uint16)
    I64, I = ctypes.c_int64, ctypes.c_int
    _check(lib().vqo_vq_gemm_a(_p(_u16(x)), _p(w), _p(_u16(cb)), _p(y), I64(M), I64(K), I64(Nc), I(E), I(ratio)))
    return y.view(np.float16)


def gemm_nt(x, w) -> np.ndarray:
    x = np.ascontiguousarray(x); w = np.ascontiguousarray(w)
    M, K = x.shape
    N = w.shape[0]
    y = np.empty((M, N), dtype=np.uint16)
    I64 = ctypes.c_int64
    _check(lib().vqo_gemm_nt(_p(_u16(x)), _p(_u16(w)), _p(y), I64(M), I64(K), I64(N)))
    return y.view(np.float16)


def gemm_nn(x, w) -> np.ndarray:
    x = np.ascontiguousarray(x); w = np.ascontiguousarray(w)
    M, K = x.shape
    N = w.shape[1]
    y = np.empty((M, N), dtype=np.uint16)
    I64 = ctypes.c_int64
    _check(lib().vqo_gemm_nn(_p(_u16(x)), _p(_u16(w)), _p(y), I64(M), I64(K), I64(N)))
    return y.view(np.float16)


def encode_b(w, codebook, code_bits: int) -> np.ndarray:
    """Nearest-codeword codes [N, K/v] of W [N,K] fp16 (fp32 fused-multiply-add distances,
    lowest index on ties)."""
    w = np.ascontiguousarray(w)
    cb = _cb3(codebook)
    G, E, v = cb.shape
    N, K = w.shape
    out = np.empty((N, K // v), dtype=np.uint8 if code_bits == 8 else np.uint16)
    I64, I = ctypes.c_int64, ctypes.c_int
    _check(lib().vqo_encode_b(_p(_u16(w)), _p(_u16(cb)), _p(out), I(code_bits), I64(N), I64(K), I(v), I(E), I(G)))
    return out
