"""The entry point that allocates nothing (vqgemm_e2e_gemm_a_noalloc) against the entry point it is a
variant of (vqgemm_e2e_gemm_a with a caller-supplied workspace): same kernels, so the outputs must be
equal bit for bit - on two calls in a row, the second on a smaller input, so that what the first call
left in the library's scratch array would show."""
import numpy as np
import pytest
import torch

from oracle import vq_oracle as vo
from vq_gemm_amd import cabi
from vq_gemm_amd.problems import GEOM_A, ProblemSpec, make_problem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _problem(M, K, Nc, seed):
    spec = ProblemSpec("A", GEOM_A, M, K, 2 * Nc, 2, 256, Nc // 4, 8, codebook_std=1.0)
    return make_problem(spec, seed=seed, device=DEV)


def test_no_alloc_entry_point_matches_the_workspace_entry_point_on_two_calls_in_a_row():
    calls = 0
    # first the reference's own shape (10 MiB of dequantised weights), then a smaller and ragged one
    shapes = [(2048, 4096, 640), (130, 96, 64)]
    for variant in (cabi.VARIANT_TWOPASS, cabi.VARIANT_AUTO):
        for i, (M, K, Nc) in enumerate(shapes):
            print("no-alloc", cabi.VARIANT_NAMES[variant], M, K, Nc, flush=True)
            x, w, cb = _problem(M, K, Nc, seed=20 + i)
            ws = torch.empty(K, 2 * Nc, dtype=torch.float16, device=DEV)
            want = cabi.e2e_gemm_a(x, w, cb, variant=variant, workspace=ws)
            out = torch.full((M, 2 * Nc), float("nan"), dtype=torch.float16, device=DEV)
            torch.cuda.synchronize()
            free_before, _ = torch.cuda.mem_get_info()   # device memory, whoever allocates it
            got = cabi.e2e_gemm_a_noalloc(x, w, cb, out, variant=variant)
            torch.cuda.synchronize()
            # (the very first call on a device looks the array up, which makes the runtime load the code object
            # that holds it: from the second call on the device's free memory does not move)
            assert calls == 0 or torch.cuda.mem_get_info()[0] == free_before
            calls += 1
            assert torch.equal(got, want), (variant, M, K, Nc)
            if i == 1:
                # and against the oracle, so that "equal" is not two wrong answers
                ref = vo.vq_gemm_a(x.cpu().numpy(), w.cpu().numpy(), cb.cpu().numpy(), acc=np.float64)
                e1, _ = vo.rel_err(got.cpu().numpy(), ref)
                assert e1 <= 2e-3, e1


def test_no_alloc_entry_point_refuses_what_does_not_fit_and_bad_arguments():
    # 4096 x 4096 dequantised weights = 32 MiB > 16 MiB, whichever route the shape would take
    x, w, cb = _problem(16, 4096, 2048, seed=1)
    out = torch.empty(16, 4096, dtype=torch.float16, device=DEV)
    with pytest.raises(cabi.VqGemmError) as ei:
        cabi.e2e_gemm_a_noalloc(x, w, cb, out)
    assert ei.value.code == -6
    x, w, cb = _problem(16, 64, 16, seed=2)
    out = torch.empty(16, 32, dtype=torch.float16, device=DEV)
    with pytest.raises(cabi.VqGemmError) as ei:
        cabi.e2e_gemm_a_noalloc(x, w, cb, out, variant=99)
    assert ei.value.code == -4
    # under stream capture: the call records its kernels and allocates nothing
    xs, ws_, cbs = _problem(64, 128, 32, seed=3)
    outs = torch.zeros(64, 64, dtype=torch.float16, device=DEV)
    want = cabi.e2e_gemm_a(xs, ws_, cbs, variant=cabi.VARIANT_TWOPASS)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        cabi.e2e_gemm_a_noalloc(xs, ws_, cbs, outs, variant=cabi.VARIANT_TWOPASS)   # first call outside capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            cabi.e2e_gemm_a_noalloc(xs, ws_, cbs, outs, variant=cabi.VARIANT_TWOPASS)
        for _ in range(3):
            outs.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(outs, want)
