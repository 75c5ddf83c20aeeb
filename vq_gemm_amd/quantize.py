"""Vector quantiser for geometry B: fp16 weights -> codes + codebooks the GEMM path consumes.

The reference only ever multiplies random codes (its harness draws them, bench.py:84); this is
the step before the path for real weights.  Plain Lloyd iterations per codebook block: the
assignment step (by far the heaviest: every vector against every entry) runs in the library's HIP
encoder (vqgemm_encode_b), the centroid update is a handful of torch reductions on the device.
Nothing here runs on the CPU and nothing falls back to it.

`residual_quantize` is the additive ("residual") mode the reference names in an unused macro
(`RESIDUAL`, strategy_1/src.cu:18-19) and never implements: W ~ sum over stages s of
codebook_s[codes_s], stage s quantising what the stages before it left.  It needs no kernel of its
own: X.(W_0 + W_1).T = [X, X].[W_0, W_1].T, so the stages are laid side by side along K - codes
[N, S*K/vec] with stage s's indices offset by s*entries into one merged codebook of S*entries
vectors - and the fused GEMM multiplies them against X repeated S times along K, all stages
accumulating in the same fp32 sums.
"""
from __future__ import annotations

from . import cabi


def kmeans_quantize(w, vec: int, entries: int, n_codebooks: int = 1, iters: int = 10, seed: int = 0):
    """Quantise W [N,K] (fp16, on the GPU) with `n_codebooks` codebooks of `entries` vectors of
    length `vec`; codebook g serves rows [g*N/G, (g+1)*N/G).

    Returns (codes [N, K/vec] uint8 or uint16, codebook [G, entries, vec] fp16, history) where
    history[i] is the mean squared error per element after assignment i (fp16 codebooks as stored).
    The final codes are the nearest entries of the returned codebook.
    """
    import torch

    if w.dtype != torch.float16 or w.dim() != 2 or not w.is_cuda:
        raise ValueError("w must be a 2-D fp16 tensor on the GPU")
    N, K = w.shape
    if K % vec or N % n_codebooks:
        raise ValueError("K must be a multiple of vec and N of n_codebooks")
    w = w.contiguous()
    G, J = n_codebooks, K // vec
    per_cb = (N // G) * J                                     # vectors per codebook block
    vectors = w.view(G, per_cb, vec)
    gen = torch.Generator(device="cpu").manual_seed(seed)
    # initial entries: distinct random vectors of the block (with repetition when the block is small)
    if per_cb >= entries:
        pick = torch.stack([torch.randperm(per_cb, generator=gen)[:entries] for _ in range(G)])
    else:
        pick = torch.randint(0, per_cb, (G, entries), generator=gen)
    pick = pick.to(w.device)
    codebook = torch.gather(vectors, 1, pick[:, :, None].expand(G, entries, vec)).contiguous()
    code_bits = 8 if entries <= 256 else 16
    vf = vectors.float()
    history = []
    codes = None
    for it in range(iters + 1):
        codes = cabi.encode_b(w, codebook, code_bits)
        idx = codes.view(G, per_cb).to(torch.int64)
        recon = torch.gather(codebook.float(), 1, idx[:, :, None].expand(G, per_cb, vec))
        history.append(float(((recon - vf) ** 2).mean()))
        if it == iters:
            break
        sums = torch.zeros(G, entries, vec, dtype=torch.float32, device=w.device)
        sums.scatter_add_(1, idx[:, :, None].expand(G, per_cb, vec), vf)
        counts = torch.zeros(G, entries, dtype=torch.float32, device=w.device)
        counts.scatter_add_(1, idx, torch.ones_like(idx, dtype=torch.float32))
        mean = sums / counts.clamp(min=1.0)[:, :, None]
        # an entry nothing was assigned to keeps its value
        codebook = torch.where(counts[:, :, None] > 0, mean, codebook.float()).half().contiguous()
    return codes, codebook, history


def residual_quantize(w, vec: int, entries: int, stages: int = 2, n_codebooks: int = 1, iters: int = 10, seed: int = 0):
    """Additive quantisation of W [N,K] (fp16, on the GPU) in `stages` rounds of `kmeans_quantize`,
    each on the residual of the rounds before it.

    Returns (codes [N, stages*K/vec], codebook [G, stages*entries, vec] fp16, history): columns
    [s*K/vec, (s+1)*K/vec) of the codes belong to stage s and index rows [s*entries, (s+1)*entries)
    of the merged codebook; uint8 while stages*entries <= 256, else uint16.  history[s] is the mean
    squared error per element of the sum of stages 0..s against W.  The layer multiplies them against
    X repeated `stages` times along K (`vq_gemm_amd.nn.VQLinear(..., k_repeat=stages)`).
    """
    import torch

    if stages < 1:
        raise ValueError("stages must be at least 1")
    if stages * entries > 65536:
        raise ValueError("stages * entries must fit 16-bit codes")
    if w.dtype != torch.float16 or w.dim() != 2 or not w.is_cuda:
        raise ValueError("w must be a 2-D fp16 tensor on the GPU")
    target = w.float()
    approx = torch.zeros_like(target)
    wide = stages * entries > 256
    all_codes, all_books, history = [], [], []
    for s in range(stages):
        residual = (target - approx).half().contiguous()
        codes, codebook, _ = kmeans_quantize(residual, vec, entries, n_codebooks, iters, seed + s)
        approx += cabi.dequant_b(codes, codebook).float()
        history.append(float(((approx - target) ** 2).mean()))
        all_codes.append(codes.to(torch.int32) + s * entries)
        all_books.append(codebook)
    merged = torch.cat(all_codes, dim=1)
    # (not every build converts to uint16 directly: narrow to int16, same bits)
    merged = merged.to(torch.int16).view(torch.uint16) if wide else merged.to(torch.uint8)
    return merged.contiguous(), torch.cat(all_books, dim=1).contiguous(), history


def interleave_gate_up(gate, up):
    """Rows of a gate/up projection pair in the order the gated epilogue expects (`vqgemm_e2e_gemm_b_gated`):
    rows 32g .. 32g+15 of the result are gate rows 16g .. 16g+15, rows 32g+16 .. 32g+31 the up rows of the same
    numbers.  Works on weights (before quantising), on codes, and on biases; both need a multiple of 16 rows."""
    import torch
    if gate.shape != up.shape or gate.shape[0] % 16 != 0:
        raise ValueError("gate and up must have the same shape and a multiple of 16 rows")
    h = gate.shape[0]
    rest = gate.shape[1:]
    return torch.stack([gate.reshape(h // 16, 16, *rest), up.reshape(h // 16, 16, *rest)], dim=1).reshape(2 * h, *rest).contiguous()
