"""Vector quantiser for geometry B: fp16 weights -> codes + codebooks the GEMM path consumes.

The reference only ever multiplies random codes (its harness draws them, bench.py:84); this is
the step before the path for real weights.  Plain Lloyd iterations per codebook block: the
assignment step (by far the heaviest: every vector against every entry) runs in the library's HIP
encoder (vqgemm_encode_b), the centroid update is a handful of torch reductions on the device.
Nothing here runs on the CPU and nothing falls back to it.
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
