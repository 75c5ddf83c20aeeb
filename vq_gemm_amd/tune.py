"""Times every kernel variant on one geometry-B shape and shows what the automatic choice picks:

    python -m vq_gemm_amd.tune M K N [vec entries codebooks code_bits]

The choice between the kernels rests on cost models fitted to measurements on one MI355X; this
prints, for the box at hand, the time of each variant that accepts the shape (launches replayed
from a HIP graph), the variant `VQGEMM_VARIANT_AUTO` resolves to, its distance from the fastest,
and the hipBLASLt fp16 GEMM on the dequantised weights beside them.  Inputs are synthetic
(X ~ N(0,1), uniform codes, codebooks ~ N(0, 0.02)), as in the bench.
"""
from __future__ import annotations

import sys

import torch

from . import cabi
from .problems import GEOM_B, ProblemSpec, make_problem


def time_graph(fn, launches: int = 20, repeats: int = 3) -> float:
    """Microseconds per launch of `fn`, replayed from a HIP graph on a side stream (default priority)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(3):
            fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(launches):
                fn()
        graph.replay()
        stream.synchronize()
        best = float("inf")
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1) / launches * 1e3)
    return best


def tune(M: int, K: int, N: int, vec: int = 8, entries: int = 256, n_codebooks: int = 1, code_bits: int = 8,
         device: str = "cuda:0", verbose: bool = True) -> dict:
    spec = ProblemSpec("tune", GEOM_B, M, K, N, vec, entries, n_codebooks, code_bits)
    x, codes, cb = make_problem(spec, seed=1, device=device)
    y = torch.empty(M, N, dtype=torch.float16, device=device)
    workspace = torch.empty(N, K, dtype=torch.float16, device=device)
    times = {}
    # a first untimed pass of the heaviest variant brings the device out of its idle clocks
    cabi.e2e_gemm_b(x, codes, cb, out=y, variant=cabi.VARIANT_TWOPASS, workspace=workspace)
    torch.cuda.synchronize()
    for variant in (cabi.VARIANT_DECODE, cabi.VARIANT_DECODE_GEMV, cabi.VARIANT_PREFILL, cabi.VARIANT_PREFILL_NARROW, cabi.VARIANT_PREFILL_SMALL,
                    cabi.VARIANT_TWOPASS, cabi.VARIANT_AUTO):
        try:
            times[variant] = time_graph(lambda: cabi.e2e_gemm_b(x, codes, cb, out=y, variant=variant, workspace=workspace))
        except cabi.VqGemmError as e:
            if e.code != -4:   # anything but "this variant does not take the shape"
                raise
    w = cabi.dequant_b(codes, cb)
    t_lib = time_graph(lambda: cabi.ref_gemm_f16(x, w, w_is_nk=True, out=y))
    picked = cabi.select_variant_b(M, K, N, vec, entries, n_codebooks, code_bits)
    forced = {v: t for v, t in times.items() if v != cabi.VARIANT_AUTO}
    fastest = min(forced, key=forced.get)
    result = {"times_us": {cabi.VARIANT_NAMES[v]: t for v, t in times.items()}, "auto_picks": cabi.VARIANT_NAMES[picked],
              "fastest": cabi.VARIANT_NAMES[fastest], "auto_over_fastest": times[cabi.VARIANT_AUTO] / forced[fastest],
              "hipblaslt_us": t_lib}
    if verbose:
        print(f"M={M} K={K} N={N} vec={vec} entries={entries} codebooks={n_codebooks} code_bits={code_bits}")
        for v, t in times.items():
            print(f"  {cabi.VARIANT_NAMES[v]:15s} {t:9.1f} us  {spec.flops / t / 1e6:8.1f} TFLOP/s")
        print(f"  {'hipBLASLt fp16':15s} {t_lib:9.1f} us  (on the dequantised weights)")
        print(f"  automatic choice: {result['auto_picks']} (the prefill variant chooses its tile itself); fastest forced "
              f"variant: {result['fastest']}; automatic / fastest = {result['auto_over_fastest']:.2f}")
    return result


def main(argv) -> int:
    if len(argv) not in (3, 7):
        print(__doc__)
        return 2
    vals = [int(a) for a in argv]
    tune(*vals)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
