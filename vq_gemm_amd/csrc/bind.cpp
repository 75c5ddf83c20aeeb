// Torch extension boundary: the two functions the reference exports from bind.cpp:3-8,
//   e2e_gemm(input, w, codebook) -> Tensor      gemm(input, w) -> Tensor
// with the same positional signatures (e2e_gemm also takes an optional `out=`), plus
// dequant(w, codebook) -> Tensor.
// This file is host-only C++: it validates tensors, allocates the result with torch's
// allocator and forwards raw pointers and the current HIP stream to the C ABI of
// libvqgemm.so (and libvqgemm_ref.so for the hipBLASLt baseline module).
//
// One source, several modules: the build compiles it once per variant with
//   -DTORCH_EXTENSION_NAME=vq_gemm_cuda_<k>  -DVQ_VARIANT=<VQGEMM_VARIANT_*>  [-DVQ_REF_MODULE]
// mirroring the reference's one-extension-per-strategy scheme (compile_kernels.py:55-68).
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include <cstdlib>

#include "../../include/vq_gemm.h"
#include "../../include/vq_gemm_ref.h"

#ifndef VQ_VARIANT
#define VQ_VARIANT VQGEMM_VARIANT_AUTO
#endif

namespace {

void check_rc(int rc, const char *what)
{
#ifdef VQ_REF_MODULE
    TORCH_CHECK(rc == 0, what, " failed: ", vqref_error_string(rc), " (code ", rc, ")");
#else
    TORCH_CHECK(rc == 0, what, " failed: ", vqgemm_error_string(rc), " (code ", rc, ")");
#endif
}

void check_dev_tensor(const torch::Tensor &t, const char *name)
{
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(t.layout() == torch::kStrided, name, " must be a dense strided tensor");
}

// Contiguous and 16-byte aligned (a contiguous view into a larger buffer may start anywhere).
torch::Tensor canon(const torch::Tensor &t)
{
    torch::Tensor c = t.contiguous();
    if ((reinterpret_cast<uintptr_t>(c.data_ptr()) & 15) != 0) c = c.clone();
    return c;
}

void *cur_stream(const torch::Tensor &t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

struct Geometry {
    bool is_a = false;
    int64_t M = 0, K = 0, N = 0;  // N = output columns
    int64_t Nc = 0;               // geometry A code columns
    int vec = 0, entries = 0, n_codebooks = 0, code_bits = 0;
};

// Geometry A: reference-native tensors (bench.py:83-85): w[K,Nc] u8, codebook[Nc/4,256,2].
// Geometry B: w[N,K/v] u8/u16, codebook [E,v] or [G,E,v].  A needs codebook.size(2) == 2,
// 256 entries and w.size(0) == K; B needs w.size(1)*v == K.
Geometry classify(const torch::Tensor &input, const torch::Tensor &w, const torch::Tensor &codebook)
{
    TORCH_CHECK(input.dim() == 2, "input must be [M,K], got ", input.dim(), " dims");
    TORCH_CHECK(w.dim() == 2, "w (codes) must be 2-D, got ", w.dim(), " dims");
    TORCH_CHECK(codebook.dim() == 2 || codebook.dim() == 3, "codebook must be [E,v] or [G,E,v]");
    TORCH_CHECK(input.scalar_type() == torch::kFloat16, "input must be float16");
    TORCH_CHECK(codebook.scalar_type() == torch::kFloat16, "codebook must be float16");
    TORCH_CHECK(w.scalar_type() == torch::kUInt8 || w.scalar_type() == torch::kUInt16,
                "w (codes) must be uint8 or uint16");
    Geometry g;
    g.M = input.size(0);
    g.K = input.size(1);
    g.code_bits = w.scalar_type() == torch::kUInt8 ? 8 : 16;
    const int64_t v = codebook.size(-1);
    const int64_t E = codebook.size(-2);
    const int64_t G = codebook.dim() == 3 ? codebook.size(0) : 1;
    const bool fits_a = g.code_bits == 8 && codebook.dim() == 3 && v == 2 && E == 256 && w.size(0) == g.K &&
                        G * 4 == w.size(1);
    const bool fits_b = v > 0 && w.size(1) * v == g.K && G > 0 && w.size(0) % G == 0;
    // Shapes with K == 2*Nc fit both; the reference-native reading wins, as this is its drop-in.
    TORCH_CHECK(fits_a || fits_b,
                "shapes fit neither layout: reference-native needs w[K,Nc] uint8 + codebook[Nc/4,256,2]; K-axis needs "
                "w[N,K/v] + codebook[E,v] or [G,E,v] with N % G == 0 (input K=", g.K, ", w=", w.sizes(),
                ", codebook=", codebook.sizes(), ")");
    g.is_a = fits_a;
    g.vec = (int)v;
    g.entries = (int)E;
    g.n_codebooks = (int)G;
    if (fits_a) {
        g.Nc = w.size(1);
        g.N = 2 * g.Nc;
    } else {
        g.N = w.size(0);
        TORCH_CHECK(E <= (int64_t(1) << g.code_bits), "codebook has more entries than the code type can address");
    }
    return g;
}

}  // namespace

#ifndef VQ_REF_MODULE

// VQGEMM_CHECK_CODES=1 in the environment: every e2e_gemm / dequant call first verifies that all
// codes are below the number of codebook entries (one extra pass over the codes and a
// synchronisation), and raises instead of returning a result that depends on the kernel.
bool check_codes_enabled()
{
    const char *e = std::getenv("VQGEMM_CHECK_CODES");
    return e && e[0] != '\0' && e[0] != '0';
}

void check_code_range(const torch::Tensor &codes, int code_bits, int64_t entries, void *stream)
{
    if (!check_codes_enabled() || codes.numel() == 0 || entries >= (int64_t(1) << code_bits)) return;
    torch::Tensor mx = torch::empty({1}, codes.options().dtype(torch::kInt32));
    check_rc(vqgemm_max_code(codes.data_ptr(), codes.numel(), code_bits, mx.data_ptr(), stream), "code-range check");
    const int64_t m = mx.item<int32_t>();
    TORCH_CHECK(m < entries, "w holds the code ", m, " but the codebook has only ", entries, " entries");
}

// e2e_gemm(input, w, codebook[, out]): `out`, when given, receives the result (fp16 [M,N], contiguous,
// on input's device) and is returned; the reference's three-argument call allocates as before.
torch::Tensor e2e_gemm(torch::Tensor input, torch::Tensor w, torch::Tensor codebook, c10::optional<torch::Tensor> out_opt)
{
    check_dev_tensor(input, "input");
    check_dev_tensor(w, "w");
    check_dev_tensor(codebook, "codebook");
    TORCH_CHECK(w.device() == input.device() && codebook.device() == input.device(),
                "input, w and codebook must be on the same device");
    const Geometry g = classify(input, w, codebook);
    c10::DeviceGuard guard(input.device());
    torch::Tensor x = canon(input), c = canon(w), cb = canon(codebook);
    torch::Tensor out;
    if (out_opt.has_value() && out_opt->defined()) {
        out = *out_opt;
        check_dev_tensor(out, "out");
        TORCH_CHECK(out.device() == input.device(), "out must be on input's device");
        TORCH_CHECK(out.scalar_type() == torch::kFloat16 && out.dim() == 2 && out.size(0) == g.M && out.size(1) == g.N,
                    "out must be float16 [", g.M, ", ", g.N, "], got ", out.sizes());
        TORCH_CHECK(out.is_contiguous() && (reinterpret_cast<uintptr_t>(out.data_ptr()) & 15) == 0,
                    "out must be contiguous and 16-byte aligned");
    } else {
        out = torch::empty({g.M, g.N}, input.options());
    }
    check_code_range(c, g.code_bits, g.entries, cur_stream(input));
    torch::Tensor ws;
    void *ws_ptr = nullptr;
    int rc;
    if (g.is_a) {
        // Reference-native tensors.  The library chooses: its fused tiled kernel where that is expected
        // to win (the reference's own scheme: codebooks in shared memory, W dequantised into a tile
        // there), otherwise the reference's two-pass strategy (strategy_1/src.cu:323-399): the bit-exact
        // dequant kernel writes W_dec[K, 2*Nc] into the scratch allocated here, then the library's own
        // tiled MFMA GEMM multiplies.  The s1 module always takes the two-pass route.
        const int variant = VQ_VARIANT == VQGEMM_VARIANT_TWOPASS ? VQGEMM_VARIANT_TWOPASS : VQGEMM_VARIANT_AUTO;
        if (variant == VQGEMM_VARIANT_TWOPASS || vqgemm_select_variant_a(g.M, g.K, g.Nc, 1) == VQGEMM_VARIANT_TWOPASS) {
            ws = torch::empty({g.K, g.N}, input.options());
            ws_ptr = ws.data_ptr();
        }
        rc = vqgemm_e2e_gemm_a(x.data_ptr(), c.data_ptr(), cb.data_ptr(), out.data_ptr(), g.M, g.K, g.Nc, variant, ws_ptr,
                               cur_stream(input));
    } else {
        if (VQ_VARIANT == VQGEMM_VARIANT_TWOPASS) {
            ws = torch::empty({g.N, g.K}, input.options());
            ws_ptr = ws.data_ptr();
        }
        rc = vqgemm_e2e_gemm_b(x.data_ptr(), c.data_ptr(), cb.data_ptr(), out.data_ptr(), g.M, g.K, g.N, g.vec,
                               g.entries, g.n_codebooks, g.code_bits, VQ_VARIANT, ws_ptr, cur_stream(input));
    }
    check_rc(rc, "e2e_gemm");
    return out;
}

torch::Tensor gemm(torch::Tensor input, torch::Tensor w)
{
    check_dev_tensor(input, "input");
    check_dev_tensor(w, "w");
    TORCH_CHECK(input.dim() == 2 && w.dim() == 2, "gemm expects input[M,K] and w[K,N]");
    TORCH_CHECK(input.scalar_type() == torch::kFloat16 && w.scalar_type() == torch::kFloat16, "gemm expects float16");
    TORCH_CHECK(input.size(1) == w.size(0), "gemm: input is [M,", input.size(1), "] but w is [", w.size(0), ",N]");
    TORCH_CHECK(w.device() == input.device(), "input and w must be on the same device");
    c10::DeviceGuard guard(input.device());
    torch::Tensor x = canon(input), ww = canon(w);
    torch::Tensor out = torch::empty({input.size(0), w.size(1)}, input.options());
    check_rc(vqgemm_gemm_f16(x.data_ptr(), ww.data_ptr(), out.data_ptr(), input.size(0), input.size(1), w.size(1),
                             cur_stream(input)),
             "gemm");
    return out;
}

// Dequantised weights: W[N,K] (K-axis layout) or W_dec[K,2*Nc] (reference-native layout).
torch::Tensor dequant(torch::Tensor w, torch::Tensor codebook)
{
    check_dev_tensor(w, "w");
    check_dev_tensor(codebook, "codebook");
    TORCH_CHECK(w.dim() == 2, "w (codes) must be 2-D");
    TORCH_CHECK(codebook.dim() == 2 || codebook.dim() == 3, "codebook must be [E,v] or [G,E,v]");
    TORCH_CHECK(codebook.scalar_type() == torch::kFloat16, "codebook must be float16");
    TORCH_CHECK(w.scalar_type() == torch::kUInt8 || w.scalar_type() == torch::kUInt16, "w must be uint8 or uint16");
    TORCH_CHECK(w.device() == codebook.device(), "w and codebook must be on the same device");
    const int64_t v = codebook.size(-1), E = codebook.size(-2);
    const int64_t G = codebook.dim() == 3 ? codebook.size(0) : 1;
    const bool is_a = w.scalar_type() == torch::kUInt8 && codebook.dim() == 3 && v == 2 && E == 256 && G * 4 == w.size(1);
    c10::DeviceGuard guard(w.device());
    torch::Tensor c = canon(w), cb = canon(codebook);
    if (!is_a) check_code_range(c, w.scalar_type() == torch::kUInt8 ? 8 : 16, E, cur_stream(w));
    auto opts = codebook.options();
    if (is_a) {
        torch::Tensor out = torch::empty({w.size(0), 2 * w.size(1)}, opts);
        check_rc(vqgemm_dequant_a(c.data_ptr(), cb.data_ptr(), out.data_ptr(), w.size(0), w.size(1), cur_stream(w)),
                 "dequant");
        return out;
    }
    TORCH_CHECK(G > 0 && w.size(0) % G == 0, "rows of w must be a multiple of the number of codebooks");
    torch::Tensor out = torch::empty({w.size(0), w.size(1) * v}, opts);
    check_rc(vqgemm_dequant_b(c.data_ptr(), cb.data_ptr(), out.data_ptr(), w.size(0), w.size(1) * v, (int)v, (int)E,
                              (int)G, w.scalar_type() == torch::kUInt8 ? 8 : 16, cur_stream(w)),
             "dequant");
    return out;
}

#else  // VQ_REF_MODULE: the library-GEMM baseline module (reference ref_gemm/cublas_gemm_fp16.cu)

torch::Tensor gemm(torch::Tensor input, torch::Tensor w)
{
    check_dev_tensor(input, "input");
    check_dev_tensor(w, "w");
    TORCH_CHECK(input.dim() == 2 && w.dim() == 2, "gemm expects input[M,K] and w[K,N]");
    TORCH_CHECK(input.scalar_type() == torch::kFloat16 && w.scalar_type() == torch::kFloat16, "gemm expects float16");
    TORCH_CHECK(input.size(1) == w.size(0), "gemm: input is [M,", input.size(1), "] but w is [", w.size(0), ",N]");
    TORCH_CHECK(w.device() == input.device(), "input and w must be on the same device");
    c10::DeviceGuard guard(input.device());
    torch::Tensor x = canon(input), ww = canon(w);
    torch::Tensor out = torch::empty({input.size(0), w.size(1)}, input.options());
    check_rc(vqref_gemm_f16(x.data_ptr(), ww.data_ptr(), out.data_ptr(), input.size(0), input.size(1), w.size(1),
                            /*w_is_nk=*/0, cur_stream(input)),
             "gemm (hipBLASLt)");
    return out;
}

// The reference's baseline module also exports e2e_gemm, as a stub that returns zeros
// (ref_gemm/cublas_gemm_fp16.cu:51-62, "Should not be called").  Same here.
torch::Tensor e2e_gemm(torch::Tensor input, torch::Tensor w, torch::Tensor codebook, c10::optional<torch::Tensor> out_opt)
{
    (void)codebook;
    (void)out_opt;
    return torch::zeros({input.size(0), w.size(1)}, input.options());
}

#endif

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("e2e_gemm", &e2e_gemm, "VQ GEMM", pybind11::arg("input"), pybind11::arg("w"), pybind11::arg("codebook"),
          pybind11::arg("out") = pybind11::none());
    m.def("gemm", &gemm, "Normal GEMM");
#ifndef VQ_REF_MODULE
    m.def("dequant", &dequant, "Codes + codebook -> fp16 weights");
#endif
}
