"""MI355X-native vector-quantized GEMM: host-side mirror of the reference's operator API.

    e2e_gemm(input, w, codebook) -> Tensor     (reference bind.cpp:3,7)
    gemm(input, w) -> Tensor                   (reference bind.cpp:4,8)
    dequant(w, codebook) -> Tensor             (the reference's dequant pass, strategy_1/src.cu:268-321)

The functions forward to the compiled torch extension (which forwards to the C ABI of
libvqgemm.so).  There is no Python or CPU fallback: if the extension is not built the import
of `vq_gemm_amd.ops` raises.
"""
__version__ = "0.1.0"
