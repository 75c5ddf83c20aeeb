"""CPU oracle for the vector-quantized GEMM path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests, the smoke check and the
bench's CPU-baseline leg may import it.  The shipped path is the HIP library; nothing
in the package falls back to this code.

It restates, in numpy, the mathematics of the reference's harness oracle
(`bench.py:37-57`: advanced-index gather from the codebook, reshape, matmul) in the two
data geometries the library serves:

* geometry A — the reference's native layout (`bench.py:83-85`):
  codes `w[K, Nc]` uint8, codebook `[Nc/4, 256, 2]` fp16,
  `W_dec[k, n*2 + r] = codebook[n // 4, w[k, n], r]`, `out[M, 2*Nc] = X @ W_dec`.
* geometry B — weights `W[N, K]` encoded along K with vector length `v`:
  codes `[N, K/v]` uint8/uint16, codebook `[E, v]` or `[G, E, v]` (one codebook per
  `N/G` consecutive output rows),
  `W[n, j*v + t] = codebook[n // (N/G)][codes[n, j]][t]`, `Y[M, N] = X @ W.T`.

The reference accumulates in fp16 (`strategy_1/src.cu:131`,
`ref_gemm/cublas_gemm_fp16.cu:45`); the contract here is fp32 accumulation rounded once
to fp16, so the GEMM functions accumulate in fp32 (and optionally fp64, which bounds the
oracle's own rounding).

Pinning status (no golden vectors exist in the reference; see tests/test_oracle.py):
  dequant_a, dequant_b  — pinned bit-exactly: hand-written known-answer cases,
                          brute-force triple loops, the C restatement, torch advanced
                          indexing written the way `bench.py:46-55` writes it.
  vq_gemm_a, vq_gemm_b, gemm — pinned: integer-valued known answers computed by hand,
                          one-hot identities, fp64 cross-accumulation, the C restatement.
  silu_mul              — pinned: closed-form values at 0, 1 and +-20, the tanh form of the
                          same function.
  pack_codes_b          — no counterpart in the reference (its w tensor is used as generated,
                          `bench.py:84`); a permutation defined by the library's header, pinned
                          by a hand-written known answer, by an element-by-element loop over the
                          header's formula, by pack/unpack round trips and - on the GPU - by the
                          fused GEMM reading W back bit-exactly through the packed matrix.
"""
from __future__ import annotations

import numpy as np

CODEBOOKS_PER_GROUP_A = 4  # reference: one codebook per 4 code columns (bench.py:40)


def _as_cb3(codebook: np.ndarray) -> np.ndarray:
    cb = np.asarray(codebook)
    if cb.ndim == 2:
        cb = cb[None]
    if cb.ndim != 3:
        raise ValueError("codebook must be [E,v] or [G,E,v]")
    return cb


def dequant_b(codes: np.ndarray, codebook: np.ndarray) -> np.ndarray:
    """Geometry B dequantisation: returns W[N, K] with the codebook's dtype.

    W[n, j*v + t] = codebook[n // (N/G)][codes[n, j]][t]   (pure indexing, bit-exact).
    """
    codes = np.asarray(codes)
    cb = _as_cb3(codebook)
    G, E, v = cb.shape
    N, J = codes.shape
    if N % G != 0:
        raise ValueError("N must be a multiple of the number of codebooks")
    idx = codes.astype(np.int64)
    if idx.size and (idx.min() < 0 or idx.max() >= E):
        raise ValueError("code out of range")
    g = (np.arange(N, dtype=np.int64) // (N // G))[:, None]        # [N,1]
    w = cb[g, idx]                                                  # [N,J,v]
    return np.ascontiguousarray(w.reshape(N, J * v))


def dequant_a(w: np.ndarray, codebook: np.ndarray) -> np.ndarray:
    """Geometry A dequantisation (`bench.py:37-55`): returns W_dec[K, Nc*ratio].

    W_dec[k, n*ratio + r] = codebook[n // 4, w[k, n], r].
    """
    w = np.asarray(w)
    cb = np.asarray(codebook)
    if cb.ndim != 3:
        raise ValueError("geometry A codebook must be [Nc/4, E, ratio]")
    K, Nc = w.shape
    if Nc % CODEBOOKS_PER_GROUP_A != 0 or cb.shape[0] * CODEBOOKS_PER_GROUP_A != Nc:
        raise ValueError("geometry A needs codebook.shape[0]*4 == code columns")
    idx = w.astype(np.int64)
    if idx.size and idx.max() >= cb.shape[1]:
        raise ValueError("code out of range")
    row = (np.arange(Nc, dtype=np.int64) // CODEBOOKS_PER_GROUP_A)[None, :]  # [1,Nc]
    dec = cb[np.broadcast_to(row, (K, Nc)), idx]                    # [K,Nc,ratio]
    return np.ascontiguousarray(dec.reshape(K, Nc * cb.shape[2]))


def _matmul(x: np.ndarray, wt: np.ndarray, acc) -> np.ndarray:
    # x [M,K], wt [K,N]; accumulate in `acc`, round once to fp16.
    return (x.astype(acc) @ wt.astype(acc)).astype(np.float16)


def vq_gemm_b(x, codes, codebook, acc=np.float32) -> np.ndarray:
    """Y[M,N] = X[M,K] @ dequant_b(codes, codebook).T, accumulated in `acc`, fp16 out."""
    w = dequant_b(codes, codebook)
    x = np.asarray(x)
    if x.shape[1] != w.shape[1]:
        raise ValueError("K mismatch")
    return _matmul(x, w.T, acc)


def vq_gemm_a(x, w, codebook, acc=np.float32) -> np.ndarray:
    """out[M, 2*Nc] = X[M,K] @ dequant_a(w, codebook)  (`bench.py:55-56`)."""
    dec = dequant_a(w, codebook)
    x = np.asarray(x)
    if x.shape[1] != dec.shape[0]:
        raise ValueError("K mismatch")
    return _matmul(x, dec, acc)


def gemm(x, w, acc=np.float32) -> np.ndarray:
    """Plain control GEMM `o[M,N] = input[M,K] @ w[K,N]` (`ref_gemm/cublas_gemm_fp16.cu:36-46`)."""
    x = np.asarray(x)
    w = np.asarray(w)
    if x.shape[1] != w.shape[0]:
        raise ValueError("K mismatch")
    return _matmul(x, w, acc)


def rel_err(y: np.ndarray, ref: np.ndarray, floor_frac: float = 1e-2):
    """Error figures used by every GEMM parity check.

    Returns (max |y-ref| / max(|ref|, tau), max|y-ref| / max|ref|) with
    tau = floor_frac * rms(ref): outputs near zero would otherwise make the
    per-element relative error unbounded whatever the accumulation precision.
    """
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if ref.size == 0:
        return 0.0, 0.0
    diff = np.abs(y - ref)
    rms = float(np.sqrt(np.mean(ref * ref)))
    tau = max(floor_frac * rms, 1e-30)
    e1 = float(np.max(diff / np.maximum(np.abs(ref), tau)))
    e2 = float(np.max(diff) / max(float(np.max(np.abs(ref))), 1e-30))
    return e1, e2


def encode_b_distances(w: np.ndarray, codebook: np.ndarray) -> np.ndarray:
    """Squared distances [N, J, E] in float64 between every vector of W [N,K] and every entry of
    its row's codebook: the brute-force statement the nearest-codeword encoder is checked against
    (the encoder itself accumulates in float32, so it is compared through these distances, not
    through an argmin that could differ on near-ties)."""
    w = np.asarray(w)
    cb = _as_cb3(codebook)
    G, E, v = cb.shape
    N, K = w.shape
    if N % G != 0 or K % v != 0:
        raise ValueError("N must be a multiple of the number of codebooks and K of the vector length")
    wv = w.astype(np.float64).reshape(N, K // v, 1, v)
    g = np.arange(N, dtype=np.int64) // (N // G)
    books = cb.astype(np.float64)[g][:, None, :, :]      # [N,1,E,v]
    return ((wv - books) ** 2).sum(axis=-1)


def silu_mul(gate_up: np.ndarray) -> np.ndarray:
    """out[m, n] = silu(a[m, n]) * a[m, N + n] for a [M, 2N] fp16, silu(g) = g / (1 + exp(-g)), in
    float64 with one rounding to fp16 (the element-wise pass behind a gate/up projection pair; no
    counterpart in the reference).  Pinned in tests/test_oracle.py by known values and identities."""
    a = np.asarray(gate_up)
    n = a.shape[1] // 2
    g = a[:, :n].astype(np.float64)
    u = a[:, n:].astype(np.float64)
    with np.errstate(over="ignore"):
        return (g / (1.0 + np.exp(-g)) * u).astype(np.float16)


def interleave_gate_up(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """The row order of a gate/up pair under the gated epilogue: rows 32g .. 32g+15 of the result are gate rows
    16g .. 16g+15, rows 32g+16 .. 32g+31 the up rows of the same numbers (first axis; a multiple of 16 rows each).
    Works on codes, weights or biases alike.  No counterpart in the reference."""
    gate, up = np.asarray(gate), np.asarray(up)
    if gate.shape != up.shape or gate.shape[0] % 16 != 0:
        raise ValueError("gate and up must have the same shape and a multiple of 16 rows")
    h = gate.shape[0]
    rest = gate.shape[1:]
    return np.stack([gate.reshape(h // 16, 16, *rest), up.reshape(h // 16, 16, *rest)], axis=1).reshape(2 * h, *rest)


def gated_gemm_b(x, codes, codebook, bias=None) -> np.ndarray:
    """y[m, 16g + r] = silu(P[m, 32g + r]) * P[m, 32g + 16 + r] with P = X . W^T (+ bias) in float64, W dequantised
    from interleaved gate/up rows (see interleave_gate_up); one rounding to fp16.  The math behind
    vqgemm_e2e_gemm_b_gated; no counterpart in the reference (its kernels store the plain product,
    strategy_2/bsz128/src.cu:163-177).  Pinned in tests/test_oracle.py by a loop over the definition and by the
    element-wise silu_mul on the de-interleaved product."""
    w = dequant_b(codes, codebook).astype(np.float64)
    if w.shape[0] % 32 != 0:
        raise ValueError("the interleaved W needs a multiple of 32 rows")
    p = np.asarray(x).astype(np.float64) @ w.T
    if bias is not None:
        p = p + np.asarray(bias).astype(np.float64)[None, :]
    m, n = p.shape
    pg = p.reshape(m, n // 32, 2, 16)
    g, u = pg[:, :, 0, :].reshape(m, n // 2), pg[:, :, 1, :].reshape(m, n // 2)
    with np.errstate(over="ignore"):
        return (g / (1.0 + np.exp(-g)) * u).astype(np.float16)


def pack_lane_bytes(vec: int, code_bytes: int) -> int:
    """Bytes of codes one lane of the decode kernel loads at a time: 16, or 8 where four lanes'
    16 bytes would cover more than the 256 k a wave owns (8-vectors with 8-bit codes)."""
    return 8 if (16 // code_bytes) * vec * 4 > 256 else 16


def pack_codes_b(codes: np.ndarray, vec: int, inverse: bool = False) -> np.ndarray:
    """The decode kernel's packed code layout (include/vq_gemm.h, vqgemm_pack_codes_b).

    packed[n//16][s][t][q][n%16][c] = codes[n][(s*256 + t*kw)//vec + q*cpl + c], flattened in that
    order and returned with the shape of `codes`; cpl = codes per lane load, kw = 4*cpl*vec.
    """
    codes = np.asarray(codes)
    N, J = codes.shape
    K = J * vec
    if K % 256 != 0 or N % 16 != 0 or vec not in (2, 4, 8):
        raise ValueError("packed layout needs K % 256 == 0, N % 16 == 0 and vec in (2, 4, 8)")
    cpl = pack_lane_bytes(vec, codes.dtype.itemsize) // codes.dtype.itemsize
    kw = 4 * cpl * vec
    T, S, L = N // 16, K // 256, 256 // kw
    if not inverse:
        # plain [tile, r, s, t, q, c] -> packed [tile, s, t, q, r, c]
        return np.ascontiguousarray(codes.reshape(T, 16, S, L, 4, cpl).transpose(0, 2, 3, 4, 1, 5)).reshape(N, J)
    return np.ascontiguousarray(codes.reshape(T, S, L, 4, 16, cpl).transpose(0, 4, 1, 2, 3, 5)).reshape(N, J)
