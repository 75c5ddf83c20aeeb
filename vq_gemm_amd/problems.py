"""Seeded synthetic problems for the VQ-GEMM path (host logic, no GPU needed).

The reference builds its inputs in `bench.py:83-85` (randn activations, uniform uint8
codes, randn codebook) from one seed (`bench.py:33`).  The same recipe is used here, on a
CPU generator so that host and device see identical bits, in the fixed order
X -> codes -> codebook.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

GEOM_A = "A"  # reference-native: codes [K, Nc] u8, codebook [Nc/4, 256, 2], vector along N
GEOM_B = "B"  # codes [N, K/v] u8/u16, codebook [E, v] or [G, E, v], vector along K


@dataclass(frozen=True)
class ProblemSpec:
    name: str
    geometry: str
    M: int
    K: int
    N: int              # output columns (geometry A: 2 * code columns)
    vec: int            # codeword length
    entries: int        # codebook entries E
    n_codebooks: int    # G (geometry A: code columns / 4)
    code_bits: int      # 8 or 16
    codebook_std: float = 0.02
    codebook_3d: Optional[bool] = None   # force a [G,E,v] tensor even when G == 1

    @property
    def code_dtype(self):
        return torch.uint8 if self.code_bits == 8 else torch.uint16

    @property
    def codes_shape(self):
        if self.geometry == GEOM_A:
            return (self.K, self.N // self.vec)
        return (self.N, self.K // self.vec)

    @property
    def codebook_shape(self):
        if self.geometry == GEOM_A or self.n_codebooks > 1 or self.codebook_3d:
            return (self.n_codebooks, self.entries, self.vec)
        return (self.entries, self.vec)

    @property
    def flops(self) -> int:
        return 2 * self.M * self.N * self.K

    @property
    def code_bytes(self) -> int:
        r, c = self.codes_shape
        return r * c * (self.code_bits // 8)

    @property
    def codebook_bytes(self) -> int:
        return self.n_codebooks * self.entries * self.vec * 2

    @property
    def algorithmic_bytes(self) -> int:
        """codes + codebooks + X + Y, each touched once."""
        return self.code_bytes + self.codebook_bytes + 2 * self.M * self.K + 2 * self.M * self.N

    @property
    def dense_weight_bytes(self) -> int:
        return 2 * self.N * self.K


# The five measured configurations (geometry B) and the reference harness's own shape
# (geometry A, bench.py:13-15,29-30).
CONFIGS = {
    "C1": ProblemSpec("C1", GEOM_B, 16, 1024, 1024, 4, 256, 1, 8),
    "C2": ProblemSpec("C2", GEOM_B, 1, 4096, 4096, 8, 256, 1, 8),
    "C3": ProblemSpec("C3", GEOM_B, 16, 4096, 11008, 4, 4096, 1, 16),
    "C4": ProblemSpec("C4", GEOM_B, 4096, 4096, 4096, 8, 256, 32, 8),
    "C5": ProblemSpec("C5", GEOM_B, 2048, 8192, 28672, 8, 256, 56, 8),
    "REF": ProblemSpec("REF", GEOM_A, 2048, 4096, 1280, 2, 256, 160, 8, codebook_std=1.0),
}


def make_problem(spec: ProblemSpec, seed: int = 42, device: str = "cpu"):
    """Returns (x, codes, codebook) for `spec`; generated on CPU, then moved to `device`."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(spec.M, spec.K, generator=g, dtype=torch.float32).half()
    # randint has no uint16 kernel on every build: draw int32 and narrow.
    codes = torch.randint(0, spec.entries, spec.codes_shape, generator=g, dtype=torch.int32)
    codes = codes.to(spec.code_dtype)
    cb = (torch.randn(spec.codebook_shape, generator=g, dtype=torch.float32) * spec.codebook_std).half()
    if device != "cpu":
        x, codes, cb = x.to(device), codes.to(device), cb.to(device)
    return x, codes, cb
