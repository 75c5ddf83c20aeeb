/*
 * Plain-C restatement of the vector-quantized GEMM mathematics.  TEST INFRASTRUCTURE ONLY:
 * it is the checker for the HIP library, never linked into or called from the product.
 *
 * Follows the reference harness oracle bench.py:37-57 (gather from the codebook, then a
 * matrix product) for geometry A, and the same rule transposed to K-axis vectors for
 * geometry B.  Written as explicit scalar loops with its own IEEE binary16 conversion so
 * that it shares no code (and no vectorised library routine) with the numpy restatement
 * it is cross-checked against.
 *
 * The nearest-codeword encoder (vqo_encode_b) has no counterpart in the reference (which only
 * ever multiplies random codes, bench.py:84); its rule is stated here and pinned by brute force
 * in float64, exact-tie cases and the dequantise -> encode round trip.
 *
 * Pinning status: every function here is pinned by tests/test_oracle.py (hand-computed
 * known answers, identities, cross-check against the numpy restatement).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

/* ---- IEEE 754 binary16 <-> binary32, bit level, round-to-nearest-even ---- */
static float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
    if (absx >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x33000001u) /* <= 2^-25 rounds to zero */
        return sign;
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q++;
    return (uint16_t)(sign | (base + q)); /* a carry out of q correctly bumps the exponent */
}

uint16_t vqo_f2h(float f) { return f2h(f); }
float vqo_h2f(uint16_t h) { return h2f(h); }

static int64_t code_at(const void *codes, int code_bits, int64_t i)
{
    return code_bits == 8 ? (int64_t)((const uint8_t *)codes)[i]
                          : (int64_t)((const uint16_t *)codes)[i];
}

/* Geometry B: W[n, j*v+t] = cb[n / (N/G)][codes[n,j]][t].  Returns 0, or -1 on bad arguments. */
int vqo_dequant_b(const void *codes, int code_bits, const uint16_t *cb, uint16_t *w_out,
                  int64_t N, int64_t K, int v, int E, int G)
{
    if (v <= 0 || G <= 0 || K % v != 0 || N % G != 0 || (code_bits != 8 && code_bits != 16))
        return -1;
    int64_t J = K / v, rpc = N / G;
    for (int64_t n = 0; n < N; n++) {
        const uint16_t *book = cb + (n / rpc) * (int64_t)E * v;
        for (int64_t j = 0; j < J; j++) {
            int64_t c = code_at(codes, code_bits, n * J + j);
            if (c >= E)
                return -2;
            for (int t = 0; t < v; t++)
                w_out[n * K + j * v + t] = book[c * v + t];
        }
    }
    return 0;
}

/* Geometry A (bench.py:46-55): W_dec[k, n*ratio+r] = cb[n/4][w[k,n]][r]; w is [K,Nc] uint8. */
int vqo_dequant_a(const uint8_t *w, const uint16_t *cb, uint16_t *w_out,
                  int64_t K, int64_t Nc, int E, int ratio)
{
    if (Nc % 4 != 0 || ratio <= 0)
        return -1;
    for (int64_t k = 0; k < K; k++)
        for (int64_t n = 0; n < Nc; n++) {
            int64_t c = w[k * Nc + n];
            if (c >= E)
                return -2;
            for (int r = 0; r < ratio; r++)
                w_out[k * Nc * ratio + n * ratio + r] = cb[((n / 4) * (int64_t)E + c) * ratio + r];
        }
    return 0;
}

/* Y[M,N] = X[M,K] . W[N,K]^T, sequential fp32 accumulation, one rounding to fp16. */
int vqo_gemm_nt(const uint16_t *x, const uint16_t *w, uint16_t *y, int64_t M, int64_t K, int64_t N)
{
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++)
                acc += h2f(x[m * K + k]) * h2f(w[n * K + k]);
            y[m * N + n] = f2h(acc);
        }
    return 0;
}

/* o[M,N] = input[M,K] . w[K,N]  (ref_gemm/cublas_gemm_fp16.cu:36-46), fp32 accumulation. */
int vqo_gemm_nn(const uint16_t *x, const uint16_t *w, uint16_t *y, int64_t M, int64_t K, int64_t N)
{
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++)
                acc += h2f(x[m * K + k]) * h2f(w[k * N + n]);
            y[m * N + n] = f2h(acc);
        }
    return 0;
}

/* Fused statements of the two paths, without materialising W (a second, independent index walk). */
int vqo_vq_gemm_b(const uint16_t *x, const void *codes, int code_bits, const uint16_t *cb,
                  uint16_t *y, int64_t M, int64_t K, int64_t N, int v, int E, int G)
{
    if (v <= 0 || G <= 0 || K % v != 0 || N % G != 0 || (code_bits != 8 && code_bits != 16))
        return -1;
    int64_t J = K / v, rpc = N / G;
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            const uint16_t *book = cb + (n / rpc) * (int64_t)E * v;
            float acc = 0.0f;
            for (int64_t j = 0; j < J; j++) {
                int64_t c = code_at(codes, code_bits, n * J + j);
                if (c >= E)
                    return -2;
                for (int t = 0; t < v; t++)
                    acc += h2f(x[m * K + j * v + t]) * h2f(book[c * v + t]);
            }
            y[m * N + n] = f2h(acc);
        }
    return 0;
}

int vqo_vq_gemm_a(const uint16_t *x, const uint8_t *w, const uint16_t *cb, uint16_t *y,
                  int64_t M, int64_t K, int64_t Nc, int E, int ratio)
{
    if (Nc % 4 != 0 || ratio <= 0)
        return -1;
    int64_t Nout = Nc * ratio;
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < Nc; n++)
            for (int r = 0; r < ratio; r++) {
                float acc = 0.0f;
                for (int64_t k = 0; k < K; k++) {
                    int64_t c = w[k * Nc + n];
                    if (c >= E)
                        return -2;
                    acc += h2f(x[m * K + k]) * h2f(cb[((n / 4) * (int64_t)E + c) * ratio + r]);
                }
                y[m * Nout + n * ratio + r] = f2h(acc);
            }
    return 0;
}

/*
 * Nearest-codeword encoder, geometry B: codes[n,j] = argmin_e sum_t (W[n,j*v+t] - cb[g][e][t])^2.
 * The distance is accumulated in binary32 in vector order with a fused multiply-add
 * (acc = fma(d, d, acc), d = w - c in binary32); entry 0 starts as the best and a later entry
 * replaces it only when strictly closer (ties keep the lowest index, a NaN distance never wins).
 */
int vqo_encode_b(const uint16_t *w, const uint16_t *cb, void *codes_out, int code_bits,
                 int64_t N, int64_t K, int v, int E, int G)
{
    if (v <= 0 || G <= 0 || E <= 0 || K % v != 0 || N % G != 0 || (code_bits != 8 && code_bits != 16))
        return -1;
    if ((int64_t)E > ((int64_t)1 << code_bits))
        return -1;
    int64_t J = K / v, rpc = N / G;
    for (int64_t n = 0; n < N; n++) {
        const uint16_t *book = cb + (n / rpc) * (int64_t)E * v;
        for (int64_t j = 0; j < J; j++) {
            float best = 0.0f;
            int64_t arg = 0;
            for (int64_t e = 0; e < E; e++) {
                float acc = 0.0f;
                for (int t = 0; t < v; t++) {
                    float d = h2f(w[n * K + j * v + t]) - h2f(book[e * v + t]);
                    acc = fmaf(d, d, acc);
                }
                if (e == 0 || acc < best) {
                    best = acc;
                    arg = e;
                }
            }
            if (code_bits == 8)
                ((uint8_t *)codes_out)[n * J + j] = (uint8_t)arg;
            else
                ((uint16_t *)codes_out)[n * J + j] = (uint16_t)arg;
        }
    }
    return 0;
}
