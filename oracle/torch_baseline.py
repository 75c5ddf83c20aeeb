"""The reference harness's math restated with torch on the host CPU.  TEST INFRASTRUCTURE ONLY.

`bench.py:37-57` of the reference computes the expected result as an advanced-index
gather from the codebook followed by a library GEMM.  This is the same two steps on CPU
tensors (gather, then an fp32 matmul rounded to fp16), used as the reported CPU baseline
and as a third independent statement of the math in the tests.
"""
from __future__ import annotations

import time

import torch


def dequant_b(codes: torch.Tensor, codebook: torch.Tensor) -> torch.Tensor:
    cb = codebook if codebook.dim() == 3 else codebook.unsqueeze(0)
    G = cb.shape[0]
    N, J = codes.shape
    g_idx = (torch.arange(N) // (N // G)).unsqueeze(1).expand(N, J)
    # uint8/uint16 tensors cannot be used as indices (uint8 means "mask"): widen first,
    # as the reference does with w.int() (bench.py:50).
    return cb[g_idx, codes.long()].reshape(N, J * cb.shape[2])


def dequant_a(w: torch.Tensor, codebook: torch.Tensor) -> torch.Tensor:
    K, Nc = w.shape
    row_idx = (torch.arange(Nc) // 4).unsqueeze(0).expand(K, Nc)      # bench.py:46-48
    dec = codebook[row_idx, w.int()]                                   # bench.py:50-53
    return dec.reshape(K, Nc * codebook.shape[2])                      # bench.py:55


def vq_gemm_b(x, codes, codebook) -> torch.Tensor:
    w = dequant_b(codes, codebook)
    return (x.float() @ w.float().t()).half()


def vq_gemm_a(x, w, codebook) -> torch.Tensor:
    dec = dequant_a(w, codebook)
    return (x.float() @ dec.float()).half()


def timed_vq_gemm_b(x, codes, codebook, reps: int = 3):
    """Returns (best seconds for dequant, best seconds for matmul, last result)."""
    best_d = best_m = float("inf")
    y = None
    for _ in range(reps):
        t0 = time.perf_counter()
        w = dequant_b(codes, codebook)
        t1 = time.perf_counter()
        y = (x.float() @ w.float().t()).half()
        t2 = time.perf_counter()
        best_d = min(best_d, t1 - t0)
        best_m = min(best_m, t2 - t1)
    return best_d, best_m, y
