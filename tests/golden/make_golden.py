"""Writes the committed fixtures under tests/golden/.

The reference holds no golden vectors (no tests directory; its logs are git-ignored), so the
fixtures are produced by this repository's CPU oracle after it has been pinned by
tests/test_oracle.py: SHA-256 digests of the seeded inputs and of the dequantised weights,
plus a few hundred fp64-accumulated output samples.  Run from the repository root:

    python -m tests.golden.make_golden
"""
from __future__ import annotations

import hashlib
import json
import os

import numpy as np

from oracle import vq_oracle as vo
from vq_gemm_amd.problems import CONFIGS, GEOM_A, ProblemSpec, make_problem

HERE = os.path.dirname(os.path.abspath(__file__))

FIXTURE_SPECS = {
    "C1": CONFIGS["C1"],
    # the reference harness's layout (bench.py:83-85) at a size the scalar C oracle finishes instantly
    "REF_small": ProblemSpec("REF_small", GEOM_A, 32, 256, 128, 2, 256, 16, 8, codebook_std=1.0),
}


def fixture_problem(spec):
    x, codes, cb = make_problem(spec, seed=42)
    return x.numpy(), codes.numpy(), cb.numpy()


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    for name, spec in FIXTURE_SPECS.items():
        x, codes, cb = fixture_problem(spec)
        if spec.geometry == GEOM_A:
            w = vo.dequant_a(codes, cb)
            y64 = x.astype(np.float64) @ w.astype(np.float64)
        else:
            w = vo.dequant_b(codes, cb)
            y64 = x.astype(np.float64) @ w.astype(np.float64).T
        rng = np.random.default_rng(7)
        rows = np.sort(rng.choice(y64.shape[0], size=min(8, y64.shape[0]), replace=False))
        cols = np.sort(rng.choice(y64.shape[1], size=min(48, y64.shape[1]), replace=False))
        w_rows = np.sort(rng.choice(w.shape[0], size=min(8, w.shape[0]), replace=False))
        w_cols = np.sort(rng.choice(w.shape[1], size=min(32, w.shape[1]), replace=False))
        np.savez(os.path.join(HERE, f"{name}.npz"), sample_rows=rows, sample_cols=cols,
                 y_samples_f64=y64[rows][:, cols], w_rows=w_rows, w_cols=w_cols,
                 w_samples=w[w_rows][:, w_cols])
        meta = {"spec": {k: getattr(spec, k) for k in ("geometry", "M", "K", "N", "vec", "entries", "n_codebooks", "code_bits", "codebook_std")},
                "seed": 42,
                "sha256": {"x": _sha(x), "codes": _sha(codes), "codebook": _sha(cb), "w_dequant": _sha(w)}}
        with open(os.path.join(HERE, f"{name}.json"), "w") as f:
            json.dump(meta, f, indent=1, sort_keys=True)
        print(name, "written")


if __name__ == "__main__":
    main()
