"""ctypes view of the C ABI (include/vq_gemm.h, include/vq_gemm_ref.h).

Used by the parity tests and the bench to drive libvqgemm.so directly with device pointers
taken from torch tensors (torch is only the allocator here).  Loading fails loudly when the
library has not been built; nothing falls back to a CPU implementation.
"""
from __future__ import annotations

import ctypes
import os
import sys
import re

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
_INCLUDE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")

(VARIANT_AUTO, VARIANT_GENERIC, VARIANT_DECODE, VARIANT_PREFILL, VARIANT_TWOPASS, VARIANT_PREFILL_NARROW,
 VARIANT_PREFILL_SMALL, VARIANT_DECODE_PACKED, VARIANT_DECODE_GEMV, VARIANT_PREFILL_SPLITK) = range(10)
VARIANT_NAMES = {0: "auto", 1: "generic", 2: "decode", 3: "prefill", 4: "twopass", 5: "prefill_narrow", 6: "prefill_small",
                 7: "decode_packed", 8: "decode_gemv", 9: "prefill_splitk"}

_I64, _I32, _P = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p

_SIGNATURES = {
    "vqgemm_e2e_gemm_b": (ctypes.c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _P, _P]),
    "vqgemm_e2e_gemm_b_bias": (ctypes.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _P, _P]),
    "vqgemm_e2e_gemm_b_gated": (ctypes.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _P, _P]),
    "vqgemm_e2e_gemm_b_ws": (ctypes.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _P, _I64, _P]),
    "vqgemm_workspace_bytes_b": (_I64, [_I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32]),
    "vqgemm_e2e_gemm_a": (ctypes.c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I32, _P, _P]),
    "vqgemm_e2e_gemm_a_noalloc": (ctypes.c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I32, _P]),
    "vqgemm_dequant_b": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _I32, _I32, _I32, _I32, _P]),
    "vqgemm_dequant_a": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _P]),
    "vqgemm_encode_b": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _I32, _I32, _I32, _I32, _P]),
    "vqgemm_pack_codes_b": (ctypes.c_int, [_P, _P, _I64, _I64, _I32, _I32, _I32, _P]),
    "vqgemm_decode_packed_supports": (ctypes.c_int, [_I64, _I64, _I64, _I32, _I32, _I32, _I32]),
    "vqgemm_gemm_f16": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _I64, _P]),
    "vqgemm_silu_mul": (ctypes.c_int, [_P, _P, _I64, _I64, _P]),
    "vqgemm_max_code": (ctypes.c_int, [_P, _I64, _I32, _P, _P]),
    "vqgemm_select_variant_b": (ctypes.c_int, [_I64, _I64, _I64, _I32, _I32, _I32, _I32]),
    "vqgemm_select_variant_a": (ctypes.c_int, [_I64, _I64, _I64, _I32]),
    "vqgemm_tuning_count": (ctypes.c_int, []),
    "vqgemm_tuning_name": (ctypes.c_char_p, [ctypes.c_int]),
    "vqgemm_tuning_get": (ctypes.c_int, [ctypes.c_char_p, ctypes.POINTER(ctypes.c_double)]),
    "vqgemm_tuning_set": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_double]),
    "vqgemm_tuning_load": (ctypes.c_int, [ctypes.c_char_p]),
    "vqgemm_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "vqgemm_version": (ctypes.c_int, []),
}
_REF_SIGNATURES = {
    "vqref_gemm_f16": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _I64, _I32, _P]),
    "vqref_tuning_info": (ctypes.c_int, [_I64, _I64, _I64, _I32, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
                                         ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]),
    "vqref_error_string": (ctypes.c_char_p, [ctypes.c_int]),
}

_lib = None
_ref = None


def declared_symbols(header: str):
    """Function names declared in include/<header> (parsed from the header text)."""
    text = open(os.path.join(_INCLUDE_DIR, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vq(?:gemm|ref)_\w+)\s*\(", text)))


def _load(name, sigs):
    path = os.path.join(_LIB_DIR, name)
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it first (python compile_kernels.py build_ext --inplace); "
                          "there is no CPU fallback")
    lib = ctypes.CDLL(path)
    for fn, (res, args) in sigs.items():
        f = getattr(lib, fn)
        f.restype = res
        f.argtypes = args
    return lib


TUNING_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuning.json")


_tuning_file = None  # the file of constants the library was handed at load, if any


def lib():
    """The C-ABI library.  When `vq_gemm_amd/tuning.json` exists (written by `python -m vq_gemm_amd.tune --fit
    --write`), VQGEMM_TUNING_FILE is not set (the library reads that one by itself) and VQGEMM_NO_PACKAGE_TUNING is not
    set either, the file is handed to the library once, here, through `vqgemm_tuning_load`; `tuning_file()` says
    which file, if any, is in force."""
    global _lib, _tuning_file
    if _lib is None:
        loaded = _load("libvqgemm.so", _SIGNATURES)
        env = os.environ.get("VQGEMM_TUNING_FILE")
        if env:
            _tuning_file = env
        elif not os.environ.get("VQGEMM_NO_PACKAGE_TUNING") and os.path.exists(TUNING_FILE):
            if loaded.vqgemm_tuning_load(TUNING_FILE.encode()) >= 0:
                _tuning_file = TUNING_FILE
                print(f"vq_gemm_amd: cost-model constants from {TUNING_FILE}", file=sys.stderr)
        _lib = loaded
    return _lib


def tuning_file():
    """Path of the file of cost-model constants in force (VQGEMM_TUNING_FILE, or the package's own tuning.json), or
    None when the compiled-in table is."""
    lib()
    return _tuning_file


def tuning() -> dict:
    """The cost-model constants the automatic kernel choice currently uses."""
    out = {}
    v = ctypes.c_double(0)
    for i in range(lib().vqgemm_tuning_count()):
        name = lib().vqgemm_tuning_name(i)
        if lib().vqgemm_tuning_get(name, ctypes.byref(v)) == 0:
            out[name.decode()] = v.value
    return out


tuning_generation = 0  # steps with every change of the table: what callers key cached kernel choices by


def set_tuning(**constants) -> None:
    global tuning_generation
    tuning_generation += 1
    for name, value in constants.items():
        rc = lib().vqgemm_tuning_set(name.encode(), float(value))
        if rc != 0:
            raise VqGemmError(rc, f"vqgemm_tuning_set({name})")


def ref_lib():
    global _ref
    if _ref is None:
        _ref = _load("libvqgemm_ref.so", _REF_SIGNATURES)
    return _ref


class VqGemmError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what} failed with code {code}: {lib().vqgemm_error_string(code).decode()}")


def _ptr(t):
    """Device address of a tensor (None passes through).  The library dereferences these on the GPU, so
    anything but a contiguous tensor in device memory is refused here rather than faulting there."""
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("expected a tensor in GPU memory, got one on " + str(t.device))
    if not t.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _cb_dims(codebook):
    if codebook.dim() == 2:
        return 1, codebook.shape[0], codebook.shape[1]
    return codebook.shape[0], codebook.shape[1], codebook.shape[2]


# The library dereferences raw device addresses with the sizes it is told, so everything it cannot
# check itself - dtypes, element counts, one device - is checked here, before any pointer is taken.
def _require(cond, msg):
    if not cond:
        raise ValueError(msg)


def _same_device(*tensors):
    ts = [t for t in tensors if t is not None]
    for t in ts:
        _require(t.is_cuda, "expected a tensor in GPU memory, got one on " + str(t.device))
    _require(all(t.device == ts[0].device for t in ts), "all tensors must be on one device")


def _code_bits(codes):
    import torch
    _require(codes.dtype in (torch.uint8, torch.uint16), f"codes must be uint8 or uint16, got {codes.dtype}")
    return 8 if codes.dtype == torch.uint8 else 16


def _check_f16(t, shape, name):
    import torch
    _require(t.dtype == torch.float16, f"{name} must be float16, got {t.dtype}")
    _require(tuple(t.shape) == tuple(shape), f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def _check_codebook(codebook):
    import torch
    _require(codebook.dim() in (2, 3) and codebook.dtype == torch.float16,
             "codebook must be a float16 [E, vec] or [G, E, vec] tensor")
    return _cb_dims(codebook)


def _check_workspace(workspace, n_halves):
    import torch
    if workspace is not None:
        _require(workspace.dtype == torch.float16 and workspace.numel() >= n_halves,
                 f"workspace must be float16 with at least {n_halves} elements")


def e2e_gemm_b(x, codes, codebook, variant=VARIANT_AUTO, out=None, workspace=None, bias=None):
    """Geometry B fused GEMM through the C ABI.  Tensors must be contiguous device tensors.
    `bias` (fp16 [N]) is added to the fp32 sums inside the kernel."""
    import torch
    _require(x.dim() == 2 and codes.dim() == 2, "x must be [M, K] and codes [N, K/vec]")
    G, E, v = _check_codebook(codebook)
    bits = _code_bits(codes)
    M, K = x.shape
    N = codes.shape[0]
    _check_f16(x, (M, K), "x")
    _require(codes.shape[1] * v == K, f"codes have {codes.shape[1]} columns of {v}-vectors but x has K = {K}")
    _require(N % G == 0, "rows of codes must be a multiple of the number of codebooks")
    _same_device(x, codes, codebook, out, workspace, bias)
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, N), "out")
    if variant == VARIANT_TWOPASS and workspace is None:
        workspace = torch.empty((N, K), dtype=torch.float16, device=x.device)
    _check_workspace(workspace, N * K)
    if bias is None:
        rc = lib().vqgemm_e2e_gemm_b(_ptr(x), _ptr(codes), _ptr(codebook), _ptr(out), M, K, N, v, E, G, bits, variant,
                                     _ptr(workspace), _stream())
    else:
        if bias.dtype != torch.float16 or bias.shape != (N,):
            raise ValueError("bias must be an fp16 tensor with one entry per output column")
        rc = lib().vqgemm_e2e_gemm_b_bias(_ptr(x), _ptr(codes), _ptr(codebook), _ptr(bias), _ptr(out), M, K, N, v, E, G,
                                          bits, variant, _ptr(workspace), _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_e2e_gemm_b")
    return out


def workspace_bytes_b(M, K, N, vec, entries, n_codebooks, code_bits, variant=VARIANT_AUTO) -> int:
    """Bytes of workspace `e2e_gemm_b_ws` would use for the shape with `variant` (0: none)."""
    n = lib().vqgemm_workspace_bytes_b(M, K, N, vec, entries, n_codebooks, code_bits, variant)
    if n < 0:
        raise VqGemmError(int(n), "vqgemm_workspace_bytes_b")
    return int(n)


def e2e_gemm_b_ws(x, codes, codebook, variant=VARIANT_AUTO, out=None, workspace=None, bias=None):
    """The fused GEMM with a sized workspace (a uint8 device tensor, 256-byte aligned as torch allocates it): lets the
    automatic choice split K over several workgroups per tile where that pays (medium M, few columns).  With
    `workspace=None` one of `workspace_bytes_b(...)` bytes is allocated when the variant wants one."""
    import torch
    _require(x.dim() == 2 and codes.dim() == 2, "x must be [M, K] and codes [N, K/vec]")
    G, E, v = _check_codebook(codebook)
    bits = _code_bits(codes)
    M, K = x.shape
    N = codes.shape[0]
    _check_f16(x, (M, K), "x")
    _require(codes.shape[1] * v == K, f"codes have {codes.shape[1]} columns of {v}-vectors but x has K = {K}")
    _require(N % G == 0, "rows of codes must be a multiple of the number of codebooks")
    if workspace is None:
        need = workspace_bytes_b(M, K, N, v, E, G, bits, variant) if variant in (VARIANT_AUTO, VARIANT_TWOPASS, VARIANT_PREFILL_SPLITK) else 0
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    else:
        _require(workspace.dtype == torch.uint8 and workspace.is_contiguous(), "workspace must be a contiguous uint8 tensor")
    _same_device(x, codes, codebook, out, workspace, bias)
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, N), "out")
    if bias is not None:
        _check_f16(bias, (N,), "bias")
    rc = lib().vqgemm_e2e_gemm_b_ws(_ptr(x), _ptr(codes), _ptr(codebook), _ptr(bias), _ptr(out), M, K, N, v, E, G, bits, variant,
                                    _ptr(workspace), 0 if workspace is None else workspace.numel(), _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_e2e_gemm_b_ws")
    return out


def e2e_gemm_b_gated(x, codes, codebook, variant=VARIANT_AUTO, out=None, workspace=None, bias=None):
    """The fused GEMM with the gated epilogue: `codes` [N, K/vec] hold gate and up rows interleaved in groups of 16
    (N % 32 == 0), the result is [M, N/2] = silu(gate product) * up product.  `workspace` ([M, N] fp16) lets the
    shapes of the K-sliced decode kernels run as the plain product plus the element-wise pass."""
    import torch
    _require(x.dim() == 2 and codes.dim() == 2, "x must be [M, K] and codes [N, K/vec]")
    G, E, v = _check_codebook(codebook)
    bits = _code_bits(codes)
    M, K = x.shape
    N = codes.shape[0]
    _check_f16(x, (M, K), "x")
    _require(codes.shape[1] * v == K, f"codes have {codes.shape[1]} columns of {v}-vectors but x has K = {K}")
    _require(N % 32 == 0, "the interleaved gate/up rows come in whole groups of 32")
    _require(N % G == 0, "rows of codes must be a multiple of the number of codebooks")
    _same_device(x, codes, codebook, out, workspace, bias)
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, N // 2), "out")
    if variant == VARIANT_TWOPASS and workspace is None:
        workspace = torch.empty((M, N), dtype=torch.float16, device=x.device)
    _check_workspace(workspace, M * N)
    if bias is not None:
        _check_f16(bias, (N,), "bias")
    rc = lib().vqgemm_e2e_gemm_b_gated(_ptr(x), _ptr(codes), _ptr(codebook), _ptr(bias), _ptr(out), M, K, N, v, E, G, bits,
                                       variant, _ptr(workspace), _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_e2e_gemm_b_gated")
    return out


def _check_geometry_a(w, codebook, K=None):
    import torch
    _require(w.dim() == 2 and w.dtype == torch.uint8, "w must be a uint8 [K, Nc] tensor")
    Kw, Nc = w.shape
    _require(K is None or Kw == K, f"w has {Kw} rows but x has K = {K}")
    _require(codebook.dtype == torch.float16 and tuple(codebook.shape) == (Nc // 4, 256, 2) and Nc % 4 == 0,
             f"codebook must be float16 [{Nc // 4}, 256, 2] for {Nc} code columns, got {tuple(codebook.shape)}")
    return Kw, Nc


def e2e_gemm_a(x, w, codebook, variant=VARIANT_AUTO, out=None, workspace=None):
    import torch
    _require(x.dim() == 2, "x must be [M, K]")
    M, K = x.shape
    _check_f16(x, (M, K), "x")
    _, Nc = _check_geometry_a(w, codebook, K)
    _same_device(x, w, codebook, out, workspace)
    if out is None:
        out = torch.empty((M, 2 * Nc), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, 2 * Nc), "out")
    if variant == VARIANT_TWOPASS and workspace is None:
        workspace = torch.empty((K, 2 * Nc), dtype=torch.float16, device=x.device)
    _check_workspace(workspace, K * 2 * Nc)
    rc = lib().vqgemm_e2e_gemm_a(_ptr(x), _ptr(w), _ptr(codebook), _ptr(out), M, K, Nc, variant, _ptr(workspace),
                                 _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_e2e_gemm_a")
    return out


def e2e_gemm_a_noalloc(x, w, codebook, out, variant=VARIANT_AUTO):
    """vqgemm_e2e_gemm_a_noalloc: geometry A with the library's own fixed scratch array.  `out` is required
    (the call itself allocates nothing); raises VqGemmError(-6) when W_dec would not fit the array."""
    _require(x.dim() == 2, "x must be [M, K]")
    M, K = x.shape
    _check_f16(x, (M, K), "x")
    _, Nc = _check_geometry_a(w, codebook, K)
    _same_device(x, w, codebook, out)
    _check_f16(out, (M, 2 * Nc), "out")
    rc = lib().vqgemm_e2e_gemm_a_noalloc(_ptr(x), _ptr(w), _ptr(codebook), _ptr(out), M, K, Nc, variant, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_e2e_gemm_a_noalloc")
    return out


def dequant_b(codes, codebook, out=None):
    import torch
    _require(codes.dim() == 2, "codes must be [N, K/vec]")
    N, J = codes.shape
    G, E, v = _check_codebook(codebook)
    bits = _code_bits(codes)
    _require(N % G == 0, "rows of codes must be a multiple of the number of codebooks")
    _same_device(codes, codebook, out)
    if out is None:
        out = torch.empty((N, J * v), dtype=torch.float16, device=codes.device)
    else:
        _check_f16(out, (N, J * v), "out")
    rc = lib().vqgemm_dequant_b(_ptr(codes), _ptr(codebook), _ptr(out), N, J * v, v, E, G, bits, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_dequant_b")
    return out


def encode_b(w, codebook, code_bits=None, out=None):
    """Nearest-codeword codes [N, K/vec] of W [N,K] fp16 for the given codebook(s)."""
    import torch
    _require(w.dim() == 2, "w must be [N, K]")
    N, K = w.shape
    _check_f16(w, (N, K), "w")
    G, E, v = _check_codebook(codebook)
    _require(K % v == 0 and N % G == 0, "K must be a multiple of vec and N of the number of codebooks")
    if code_bits is None:
        code_bits = 8 if E <= 256 else 16
    _require(code_bits in (8, 16), "code_bits must be 8 or 16")
    _same_device(w, codebook, out)
    if out is None:
        out = torch.empty((N, K // v), dtype=torch.uint8 if code_bits == 8 else torch.uint16, device=w.device)
    else:
        _require(_code_bits(out) == code_bits and tuple(out.shape) == (N, K // v),
                 f"out must be a {code_bits}-bit code tensor of shape {(N, K // v)}")
    rc = lib().vqgemm_encode_b(_ptr(w), _ptr(codebook), _ptr(out), N, K, v, E, G, code_bits, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_encode_b")
    return out


def pack_codes_b(codes, vec, inverse=False, out=None):
    """The code matrix [N, K/vec] re-laid for VARIANT_DECODE_PACKED (same shape and dtype; `inverse`
    restores the plain matrix)."""
    import torch
    _require(codes.dim() == 2, "codes must be [N, K/vec]")
    N, J = codes.shape
    bits = _code_bits(codes)
    _same_device(codes, out)
    if out is None:
        out = torch.empty_like(codes)
    else:
        _require(out.dtype == codes.dtype and out.shape == codes.shape, "out must match codes in dtype and shape")
    rc = lib().vqgemm_pack_codes_b(_ptr(codes), _ptr(out), N, J * vec, vec, bits, 1 if inverse else 0, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_pack_codes_b")
    return out


def max_code(codes) -> int:
    """Largest code of a uint8/uint16 code tensor (synchronises: the value is read back)."""
    import torch
    bits = _code_bits(codes)
    _same_device(codes)
    out = torch.empty(1, dtype=torch.int32, device=codes.device)
    rc = lib().vqgemm_max_code(_ptr(codes), codes.numel(), bits, _ptr(out), _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_max_code")
    return int(out.item())


def decode_packed_supports(M, K, N, vec, entries, n_codebooks, code_bits) -> bool:
    return lib().vqgemm_decode_packed_supports(M, K, N, vec, entries, n_codebooks, code_bits) == 1


def dequant_a(w, codebook, out=None):
    import torch
    K, Nc = _check_geometry_a(w, codebook)
    _same_device(w, codebook, out)
    if out is None:
        out = torch.empty((K, 2 * Nc), dtype=torch.float16, device=w.device)
    else:
        _check_f16(out, (K, 2 * Nc), "out")
    rc = lib().vqgemm_dequant_a(_ptr(w), _ptr(codebook), _ptr(out), K, Nc, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_dequant_a")
    return out


def gemm_f16(x, w, out=None):
    import torch
    _require(x.dim() == 2 and w.dim() == 2, "x must be [M, K] and w [K, N]")
    M, K = x.shape
    N = w.shape[1]
    _check_f16(x, (M, K), "x")
    _check_f16(w, (K, N), "w")
    _same_device(x, w, out)
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, N), "out")
    rc = lib().vqgemm_gemm_f16(_ptr(x), _ptr(w), _ptr(out), M, K, N, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_gemm_f16")
    return out


def silu_mul(gate_up, out=None):
    """out[M,N] = silu(gate_up[:, :N]) * gate_up[:, N:] for a contiguous fp16 [M, 2N] device tensor."""
    import torch
    _require(gate_up.dim() == 2, "expected an fp16 [M, 2N] tensor")
    M, N2 = gate_up.shape
    if N2 % 2 != 0 or gate_up.dtype != torch.float16:
        raise ValueError("expected an fp16 [M, 2N] tensor")
    _same_device(gate_up, out)
    if out is None:
        out = torch.empty((M, N2 // 2), dtype=torch.float16, device=gate_up.device)
    else:
        _check_f16(out, (M, N2 // 2), "out")
    rc = lib().vqgemm_silu_mul(_ptr(gate_up), _ptr(out), M, N2 // 2, _stream())
    if rc != 0:
        raise VqGemmError(rc, "vqgemm_silu_mul")
    return out


def ref_gemm_f16(x, w, w_is_nk=False, out=None):
    """hipBLASLt baseline: x[M,K] @ w[K,N], or x @ w[N,K].T when w_is_nk."""
    import torch
    _require(x.dim() == 2 and w.dim() == 2, "x must be [M, K] and w [K, N] or [N, K]")
    M, K = x.shape
    N = w.shape[0] if w_is_nk else w.shape[1]
    _check_f16(x, (M, K), "x")
    _check_f16(w, (N, K) if w_is_nk else (K, N), "w")
    _same_device(x, w, out)
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    else:
        _check_f16(out, (M, N), "out")
    rc = ref_lib().vqref_gemm_f16(_ptr(x), _ptr(w), _ptr(out), M, K, N, 1 if w_is_nk else 0, _stream())
    if rc != 0:
        raise RuntimeError(f"vqref_gemm_f16 failed with code {rc}: {ref_lib().vqref_error_string(rc).decode()}")
    return out


def ref_tuning_info(M, K, N, w_is_nk=False):
    """What the baseline's first call on the shape found: (answers timed, index kept, its microseconds, the
    first answer's microseconds), cold caches; None when the shape has not been run."""
    n, i = ctypes.c_int32(0), ctypes.c_int32(0)
    best, first = ctypes.c_float(0), ctypes.c_float(0)
    rc = ref_lib().vqref_tuning_info(M, K, N, 1 if w_is_nk else 0, ctypes.byref(n), ctypes.byref(i), ctypes.byref(best),
                                     ctypes.byref(first))
    if rc != 0:
        return None
    return {"candidates": n.value, "chosen": i.value, "best_us": best.value, "first_answer_us": first.value}


def select_variant_a(M, K, Nc, has_workspace=False) -> int:
    return lib().vqgemm_select_variant_a(M, K, Nc, 1 if has_workspace else 0)


def select_variant_b(M, K, N, vec, entries, n_codebooks, code_bits) -> int:
    return lib().vqgemm_select_variant_b(M, K, N, vec, entries, n_codebooks, code_bits)
