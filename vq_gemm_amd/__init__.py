"""MI355X-native vector-quantized GEMM: host-side mirror of the reference's operator API.

    e2e_gemm(input, w, codebook) -> Tensor     (reference bind.cpp:3,7)
    gemm(input, w) -> Tensor                   (reference bind.cpp:4,8)
    dequant(w, codebook) -> Tensor             (the reference's dequant pass, strategy_1/src.cu:268-321)

The three names are exported here and resolve, on first use, to `vq_gemm_amd.ops` (the compiled
torch extension modules, which forward to the C ABI of libvqgemm.so).  Importing the package itself
loads nothing, so that the build driver can import it before anything is built.  There is no Python
or CPU fallback: if the extension is not built the first call raises ImportError.
"""
__version__ = "0.2.0"

__all__ = ["e2e_gemm", "gemm", "dequant"]


def __getattr__(name):
    if name in __all__:
        from . import ops
        return getattr(ops, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
