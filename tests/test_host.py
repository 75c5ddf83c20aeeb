"""CPU-side checks of the boundary: the C-ABI libraries load and export what the headers
declare, argument validation rejects bad calls before anything touches a GPU, the torch
modules exist under the names the reference harness imports, and the workload table matches
the published byte/flop figures of the five configurations."""
import ctypes
import os

import pytest
import torch

from vq_gemm_amd import cabi, ops
from vq_gemm_amd.problems import CONFIGS, make_problem


def test_libvqgemm_exports_every_declared_symbol():
    lib = cabi.lib()
    names = cabi.declared_symbols("vq_gemm.h")
    assert {"vqgemm_e2e_gemm_b", "vqgemm_e2e_gemm_a", "vqgemm_dequant_b", "vqgemm_dequant_a", "vqgemm_gemm_f16",
            "vqgemm_select_variant_b", "vqgemm_error_string", "vqgemm_version"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.vqgemm_version() >= 100


def test_libvqgemm_ref_exports_every_declared_symbol():
    lib = cabi.ref_lib()
    names = cabi.declared_symbols("vq_gemm_ref.h")
    assert "vqref_gemm_f16" in names
    for n in names:
        assert hasattr(lib, n), n


def test_argument_validation_happens_before_any_gpu_call():
    lib = cabi.lib()
    one = ctypes.c_void_p(16)  # never dereferenced: every call below is rejected first
    call = lambda **kw: lib.vqgemm_e2e_gemm_b(one, one, one, one, kw.get("M", 1), kw.get("K", 64), kw.get("N", 16),
                                              kw.get("vec", 8), kw.get("E", 256), kw.get("G", 1), kw.get("bits", 8),
                                              kw.get("variant", 0), None, None)
    assert call(M=-1) == -2
    assert call(K=60) == -2                    # K % vec != 0
    assert call(N=10, G=4) == -2               # N % n_codebooks != 0
    assert call(bits=12) == -3
    assert call(E=257) == -3                   # 257 entries do not fit 8-bit codes
    assert call(variant=9) == -4
    assert call(M=0) == 0 and call(N=0) == 0   # empty problems succeed without a launch
    assert lib.vqgemm_e2e_gemm_b(None, one, one, one, 1, 64, 16, 8, 256, 1, 8, 0, None, None) == -1
    assert lib.vqgemm_e2e_gemm_b(ctypes.c_void_p(17), one, one, one, 1, 64, 16, 8, 256, 1, 8, 0, None, None) == -5
    assert lib.vqgemm_e2e_gemm_a(one, one, one, one, 1, 64, 6, 0, None, None) == -2   # Nc % 4 != 0
    assert lib.vqgemm_dequant_b(one, one, one, 16, 60, 8, 256, 1, 8, None) == -2
    assert lib.vqgemm_dequant_a(one, one, one, 16, 6, None) == -2
    assert lib.vqgemm_gemm_f16(one, one, one, -1, 1, 1, None) == -2
    for code in (0, -1, -2, -3, -4, -5):
        assert len(lib.vqgemm_error_string(code)) > 0


def test_variant_selection_for_the_measured_configurations():
    want = {"C1": cabi.VARIANT_DECODE, "C2": cabi.VARIANT_DECODE_GEMV, "C3": cabi.VARIANT_DECODE,
            "C4": cabi.VARIANT_PREFILL, "C5": cabi.VARIANT_PREFILL}
    for name, v in want.items():
        s = CONFIGS[name]
        assert cabi.select_variant_b(s.M, s.K, s.N, s.vec, s.entries, s.n_codebooks, s.code_bits) == v, name
    # shapes the tiled kernels cannot take fall back to the generic kernel
    assert cabi.select_variant_b(4, 36, 8, 3, 10, 1, 8) == cabi.VARIANT_GENERIC
    assert cabi.select_variant_b(4, 0, 8, 8, 256, 1, 8) == cabi.VARIANT_GENERIC
    assert cabi.select_variant_b(4, 60, 8, 8, 256, 1, 8) < 0


def test_workload_table_matches_published_figures():
    want = {"C1": (329_728, 33_554_432), "C2": (2_117_632, 33_554_432), "C3": (23_060_480, 1_442_840_576),
            "C4": (69_337_088, 137_438_953_472), "C5": (180_584_448, 962_072_674_304)}
    for name, (nbytes, flops) in want.items():
        assert CONFIGS[name].algorithmic_bytes == nbytes, name
        assert CONFIGS[name].flops == flops, name
    assert CONFIGS["REF"].codes_shape == (4096, 640) and CONFIGS["REF"].codebook_shape == (160, 256, 2)


def test_problem_generator_is_deterministic_and_in_range():
    s = CONFIGS["C1"]
    a = make_problem(s, seed=42)
    b = make_problem(s, seed=42)
    for t, u in zip(a, b):
        assert torch.equal(t, u)
    x, codes, cb = a
    assert x.dtype == torch.float16 and x.shape == (16, 1024)
    assert codes.dtype == torch.uint8 and codes.shape == (1024, 256)
    assert cb.shape == (256, 4) and abs(cb.float().std().item() - 0.02) < 2e-3
    x3, c3, cb3 = make_problem(CONFIGS["C3"].__class__("t", "B", 2, 64, 32, 4, 4096, 1, 16), seed=1)
    assert c3.dtype == torch.uint16 and int(c3.to(torch.int32).max()) < 4096


@pytest.mark.parametrize("key", ops.VARIANT_KEYS)
def test_torch_modules_exist_under_the_reference_names(key):
    mod = ops.load_module(key)
    assert mod.__name__ == f"vq_gemm_cuda_{key}"
    assert callable(mod.e2e_gemm) and callable(mod.gemm)


def test_torch_module_rejects_bad_tensors_with_runtime_error():
    mod = ops.load_module("s2_128")
    x = torch.zeros(2, 8, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        mod.e2e_gemm(x, torch.zeros(4, 1, dtype=torch.uint8), torch.zeros(256, 8, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        mod.gemm(x, torch.zeros(8, 4, dtype=torch.float16))
    with pytest.raises(KeyError):
        ops.load_module("s9")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(cabi, "_LIB_DIR", str(tmp_path))
    monkeypatch.setattr(cabi, "_lib", None)
    with pytest.raises(ImportError, match="no CPU fallback"):
        cabi.lib()
    monkeypatch.setattr(ops, "_LIB_DIR", str(tmp_path))
    monkeypatch.setattr(ops, "_modules", {})
    with pytest.raises(ImportError, match="no CPU fallback"):
        ops.load_module("s2_128")


def test_registered_op_propagates_shapes_and_has_no_cpu_implementation():
    import torch
    from vq_gemm_amd import torch_ops  # noqa: F401
    x = torch.empty(3, 5, 64, dtype=torch.float16, device="meta")
    codes = torch.empty(32, 8, dtype=torch.uint8, device="meta")
    cb = torch.empty(2, 256, 8, dtype=torch.float16, device="meta")
    y = torch.ops.vq_gemm_amd.vq_linear(x, codes, cb)
    assert y.shape == (3, 5, 32) and y.dtype == torch.float16
    with pytest.raises(ValueError):   # 64 features against 8 codes x 4
        torch.ops.vq_gemm_amd.vq_linear(x, codes, torch.empty(256, 4, dtype=torch.float16, device="meta"))
    with pytest.raises(NotImplementedError):
        torch.ops.vq_gemm_amd.vq_linear(torch.zeros(2, 64, dtype=torch.float16), torch.zeros(32, 8, dtype=torch.uint8),
                                        torch.zeros(256, 8, dtype=torch.float16))


def test_ctypes_wrappers_refuse_host_tensors():
    import torch
    from vq_gemm_amd import cabi
    x = torch.zeros(2, 64, dtype=torch.float16)
    codes = torch.zeros(32, 8, dtype=torch.uint8)
    cb = torch.zeros(256, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        cabi.e2e_gemm_b(x, codes, cb)
    with pytest.raises(ValueError):
        cabi.dequant_b(codes, cb)


def test_tuning_constants_can_be_read_set_and_loaded_from_a_file(tmp_path):
    import json
    from vq_gemm_amd import cabi
    before = cabi.tuning()
    assert {"prefill_stage_us_256x256", "decode_tile_us", "gemv_max_tiles_per_cu", "gemv_wide_min_rows_per_wave"} <= set(before)
    try:
        # the choice between the four-wave GEMV kernel and the K-sliced kernel follows the constant
        dims = (1, 4096, 16 * 256 * 2, 4, 256, 1, 8)   # one row of X, 4-vectors: two tiles per unit on a 256-CU device
        cabi.set_tuning(gemv_max_tiles_per_cu=4)
        assert cabi.select_variant_b(*dims) == cabi.VARIANT_DECODE_GEMV
        cabi.set_tuning(gemv_max_tiles_per_cu=1)
        assert cabi.select_variant_b(*dims) == cabi.VARIANT_DECODE
        path = tmp_path / "t.json"
        path.write_text(json.dumps({"device": "some name: 3", "gemv_max_tiles_per_cu": 8, "decode_tile_us": 0.5, "not_a_constant": 1}))
        assert cabi.lib().vqgemm_tuning_load(str(path).encode()) == 2
        assert cabi.tuning()["decode_tile_us"] == 0.5 and cabi.select_variant_b(*dims) == cabi.VARIANT_DECODE_GEMV
        assert cabi.lib().vqgemm_tuning_load(b"/nonexistent/file.json") == -1
        assert cabi.lib().vqgemm_tuning_set(b"no_such_constant", 1.0) == -4
        assert cabi.lib().vqgemm_tuning_set(b"decode_tile_us", -1.0) == -2
    finally:
        cabi.set_tuning(**before)
    assert cabi.tuning() == before


def test_vqlinear_codes_key_works_on_inference_tensors():
    # a module whose codes were made under torch.inference_mode(): such tensors keep no version counter
    from vq_gemm_amd.nn import VQLinear
    with torch.inference_mode():
        codes = torch.zeros(32, 32, dtype=torch.uint8)
        cb = torch.zeros(256, 8, dtype=torch.float16)
        layer = VQLinear(codes, cb)
        k1 = layer._codes_key()
    assert layer.codes.is_inference()
    assert layer._codes_key() == k1
    # an ordinary tensor: the key follows in-place updates
    layer2 = VQLinear(torch.zeros(32, 32, dtype=torch.uint8), cb.clone())
    k2 = layer2._codes_key()
    layer2.codes.add_(1)
    assert layer2._codes_key() != k2
