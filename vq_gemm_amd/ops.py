"""Loads the compiled extension modules and exposes the reference's call surface.

Variant keys are the reference's strategy names (reference compile_kernels.py:11-17,
bench.py:21-27): "s1" is the two-pass strategy, "s2_128", "s2_512", "s3_naive", "s3_wasp" are
the fused ones, "cublas_gemm" is the library-GEMM baseline (hipBLASLt here).
"""
from __future__ import annotations

import importlib.util
import os

import torch  # noqa: F401  (loads libtorch/libamdhip64 before the extension)

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
_modules = {}

VARIANT_KEYS = ("cublas_gemm", "s1", "s2_128", "s2_512", "s3_naive", "s3_wasp")
DEFAULT_VARIANT = "s2_128"


def load_module(key: str = DEFAULT_VARIANT):
    """Import vq_gemm_cuda_<key> from vq_gemm_amd/lib.  Raises if it has not been built."""
    if key not in VARIANT_KEYS:
        raise KeyError(f"unknown kernel variant {key!r}; known: {', '.join(VARIANT_KEYS)}")
    if key not in _modules:
        name = f"vq_gemm_cuda_{key}"
        path = os.path.join(_LIB_DIR, name + ".so")
        if not os.path.exists(path):
            raise ImportError(
                f"{path} is missing: build the HIP extension first "
                f"(python compile_kernels.py build_ext --inplace). There is no CPU fallback.")
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _modules[key] = mod
    return _modules[key]


def e2e_gemm(input, w, codebook, variant: str = DEFAULT_VARIANT, out=None):
    """Fused VQ GEMM; same positional arguments as the reference's e2e_gemm.  `out` (fp16 [M,N],
    contiguous, on input's device) receives the result instead of a new tensor."""
    return load_module(variant).e2e_gemm(input, w, codebook, out=out)


def gemm(input, w, variant: str = DEFAULT_VARIANT):
    """Plain fp16 GEMM input[M,K] @ w[K,N]; `variant="cublas_gemm"` selects hipBLASLt."""
    return load_module(variant).gemm(input, w)


def dequant(w, codebook, variant: str = DEFAULT_VARIANT):
    """Codes + codebook -> fp16 weights, bit-exact."""
    return load_module(variant).dequant(w, codebook)
