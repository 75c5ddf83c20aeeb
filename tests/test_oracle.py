"""Pins the CPU oracle (oracle/) before anything is compared against it.

The reference holds no golden vectors for this path (its only check is a print of the
mean/max difference, bench.py:97-103), so the oracle is pinned by what the mathematics
fixes: hand-computed known answers, brute-force index walks, identities that a dropped
term, a transposed operand or a wrong codebook index would break, and agreement of three
independently written restatements (numpy, plain C, torch advanced indexing as in
bench.py:46-56).
"""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, torch_baseline
from oracle import vq_oracle as vo

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---------------------------------------------------------------- fp16 conversion of the C oracle
def test_c_half_to_float_all_values():
    lib = c_oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.vqo_h2f(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_c_float_to_half_round_to_nearest_even():
    lib = c_oracle.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 3,
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),       # subnormal halves
        (rng.standard_normal(2000) * 7e4).astype(np.float32),        # overflow region
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  1.00048828125, 1.0009765625 + 2.0 ** -11, np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 1100, dtype=np.float32) + 0.5) / 1024.0,
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([lib.vqo_f2h(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- hand-computed known answers
def test_dequant_b_known_answer():
    # two codebooks (rows 0-1 use book 0, rows 2-3 use book 1), 3 entries, vec 2
    cb = np.array([[[1, 2], [3, 4], [5, 6]],
                   [[10, 20], [30, 40], [50, 60]]], dtype=np.float16)
    codes = np.array([[0, 2], [1, 1], [2, 0], [0, 1]], dtype=np.uint8)
    want = np.array([[1, 2, 5, 6],
                     [3, 4, 3, 4],
                     [50, 60, 10, 20],
                     [10, 20, 30, 40]], dtype=np.float16)
    for fn in (vo.dequant_b, c_oracle.dequant_b):
        assert np.array_equal(fn(codes, cb), want), fn
    got_t = torch_baseline.dequant_b(torch.from_numpy(codes), torch.from_numpy(cb)).numpy()
    assert np.array_equal(got_t, want)


def test_dequant_a_known_answer():
    # Nc = 8 code columns -> 2 codebooks (one per 4 columns), 256 entries, ratio 2.
    # entry e of book b holds (100*b + e, -(100*b + e)).
    e = np.arange(256, dtype=np.float32)
    cb = np.stack([np.stack([100 * b + e, -(100 * b + e)], axis=1) for b in range(2)]).astype(np.float16)
    w = np.array([[0, 1, 2, 3, 4, 5, 6, 7],
                  [7, 7, 7, 7, 9, 9, 9, 9]], dtype=np.uint8)
    want = np.array([[0, -0.0, 1, -1, 2, -2, 3, -3, 104, -104, 105, -105, 106, -106, 107, -107],
                     [7, -7, 7, -7, 7, -7, 7, -7, 109, -109, 109, -109, 109, -109, 109, -109]], dtype=np.float16)
    for fn in (vo.dequant_a, c_oracle.dequant_a):
        assert np.array_equal(fn(w, cb).view(np.uint16), want.view(np.uint16)), fn
    got_t = torch_baseline.dequant_a(torch.from_numpy(w), torch.from_numpy(cb)).numpy()
    assert np.array_equal(got_t.view(np.uint16), want.view(np.uint16))


def test_vq_gemm_b_known_answer_integers():
    cb = np.array([[[1, 2], [3, 4], [5, 6]],
                   [[10, 20], [30, 40], [50, 60]]], dtype=np.float16)
    codes = np.array([[0, 2], [1, 1], [2, 0], [0, 1]], dtype=np.uint8)
    x = np.array([[1, 0, 0, 0],
                  [1, 1, 1, 1],
                  [2, -1, 0, 3]], dtype=np.float16)
    # W rows: [1 2 5 6], [3 4 3 4], [50 60 10 20], [10 20 30 40]
    want = np.array([[1, 3, 50, 10],
                     [14, 14, 140, 100],
                     [2 - 2 + 18, 6 - 4 + 12, 100 - 60 + 60, 20 - 20 + 120]], dtype=np.float16)
    for fn in (vo.vq_gemm_b, c_oracle.vq_gemm_b):
        assert np.array_equal(fn(x, codes, cb), want), fn
    assert np.array_equal(vo.vq_gemm_b(x, codes, cb, acc=np.float64), want)
    got_t = torch_baseline.vq_gemm_b(torch.from_numpy(x), torch.from_numpy(codes), torch.from_numpy(cb)).numpy()
    assert np.array_equal(got_t, want)


def test_vq_gemm_a_known_answer_integers():
    e = np.arange(256, dtype=np.float32)
    cb = np.stack([np.stack([e, 2 * e], axis=1)]).astype(np.float16)          # one book: Nc = 4
    w = np.array([[1, 2, 3, 4],
                  [5, 6, 7, 8],
                  [0, 0, 1, 1]], dtype=np.uint8)                                  # K = 3
    x = np.array([[1, 1, 1], [1, -1, 2]], dtype=np.float16)
    # W_dec rows: [1 2 2 4 3 6 4 8], [5 10 6 12 7 14 8 16], [0 0 0 0 1 2 1 2]
    want = np.array([[6, 12, 8, 16, 11, 22, 13, 26],
                     [-4, -8, -4, -8, -2, -4, -2, -4]], dtype=np.float16)
    for fn in (vo.vq_gemm_a, c_oracle.vq_gemm_a):
        assert np.array_equal(fn(x, w, cb), want), fn
    got_t = torch_baseline.vq_gemm_a(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(cb)).numpy()
    assert np.array_equal(got_t, want)


# ---------------------------------------------------------------- brute force on small random inputs
def _rand_b(rng, M, K, N, v, E, G, bits):
    x = rng.standard_normal((M, K)).astype(np.float16)
    codes = rng.integers(0, E, size=(N, K // v)).astype(np.uint8 if bits == 8 else np.uint16)
    cb = (rng.standard_normal((G, E, v)) * 0.02).astype(np.float16)
    return x, codes, cb


@pytest.mark.parametrize("M,K,N,v,E,G,bits", [
    (3, 16, 8, 4, 256, 1, 8), (5, 24, 12, 8, 256, 3, 8), (2, 12, 6, 2, 7, 2, 8),
    (4, 32, 10, 4, 4096, 1, 16), (1, 40, 9, 8, 300, 3, 16), (2, 9, 4, 3, 5, 2, 8),
])
def test_dequant_b_brute_force(M, K, N, v, E, G, bits):
    rng = np.random.default_rng(K * N + v)
    _, codes, cb = _rand_b(rng, M, K, N, v, E, G, bits)
    want = np.zeros((N, K), dtype=np.float16)
    for n in range(N):                      # the defining triple loop
        for j in range(K // v):
            for t in range(v):
                want[n, j * v + t] = cb[n // (N // G)][int(codes[n, j])][t]
    for fn in (vo.dequant_b, c_oracle.dequant_b):
        assert np.array_equal(fn(codes, cb).view(np.uint16), want.view(np.uint16)), fn
    got_t = torch_baseline.dequant_b(torch.from_numpy(codes), torch.from_numpy(cb)).numpy()
    assert np.array_equal(got_t.view(np.uint16), want.view(np.uint16))


def test_dequant_a_brute_force():
    rng = np.random.default_rng(5)
    K, Nc = 7, 12
    w = rng.integers(0, 256, size=(K, Nc)).astype(np.uint8)
    cb = rng.standard_normal((Nc // 4, 256, 2)).astype(np.float16)
    want = np.zeros((K, 2 * Nc), dtype=np.float16)
    for k in range(K):
        for n in range(Nc):
            for r in range(2):
                want[k, 2 * n + r] = cb[n // 4][int(w[k, n])][r]
    for fn in (vo.dequant_a, c_oracle.dequant_a):
        assert np.array_equal(fn(w, cb).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("M,K,N,v,E,G,bits", [
    (16, 1024, 64, 4, 256, 1, 8), (1, 4096, 32, 8, 256, 1, 8), (7, 512, 48, 8, 256, 3, 8),
    (5, 256, 40, 4, 4096, 1, 16),
])
def test_gemm_restatements_agree(M, K, N, v, E, G, bits):
    """numpy fp32, numpy fp64, C (fused walk), C (dequant then matmul) and torch agree."""
    rng = np.random.default_rng(M + K + N)
    x, codes, cb = _rand_b(rng, M, K, N, v, E, G, bits)
    y32 = vo.vq_gemm_b(x, codes, cb)
    y64 = vo.vq_gemm_b(x, codes, cb, acc=np.float64)
    yc = c_oracle.vq_gemm_b(x, codes, cb)
    yc2 = c_oracle.gemm_nt(x, c_oracle.dequant_b(codes, cb))
    yt = torch_baseline.vq_gemm_b(torch.from_numpy(x), torch.from_numpy(codes), torch.from_numpy(cb)).numpy()
    assert np.array_equal(yc, yc2)          # same sequential fp32 order, two different index walks
    for y in (y32, yc, yt):
        e1, e2 = vo.rel_err(y, y64)
        assert e1 <= 2e-3 and e2 <= 1e-3, (e1, e2)


# ---------------------------------------------------------------- identities
def test_one_hot_rows_return_weight_columns_exactly():
    rng = np.random.default_rng(11)
    K, N = 64, 24
    _, codes, cb = _rand_b(rng, 1, K, N, 8, 256, 3, 8)
    x = np.eye(K, dtype=np.float16)
    w = vo.dequant_b(codes, cb)
    for fn in (vo.vq_gemm_b, c_oracle.vq_gemm_b):
        y = fn(x, codes, cb)
        assert np.array_equal(y.view(np.uint16), w.T.copy().view(np.uint16))


def test_constant_codes_and_zero_codebook():
    rng = np.random.default_rng(12)
    M, K, N, v = 4, 32, 16, 4
    x = rng.standard_normal((M, K)).astype(np.float16)
    cb = (rng.standard_normal((1, 256, v)) * 0.02).astype(np.float16)
    codes = np.full((N, K // v), 37, dtype=np.uint8)
    y = vo.vq_gemm_b(x, codes, cb)
    assert np.all(y == y[:, :1])                                  # every W row is the same
    tiled = np.tile(cb[0, 37], K // v).astype(np.float32)
    assert np.array_equal(y[:, 0], (x.astype(np.float32) @ tiled).astype(np.float16))
    assert not np.any(vo.vq_gemm_b(x, codes, np.zeros_like(cb)))


def test_entry_permutation_and_codebook_replication():
    rng = np.random.default_rng(13)
    M, K, N, v, E = 3, 48, 12, 8, 256
    x, codes, cb = _rand_b(rng, M, K, N, v, E, 1, 8)
    perm = rng.permutation(E)
    inv = np.argsort(perm)
    cb_p = cb[:, perm]                       # entry i of cb_p is old entry perm[i]
    codes_p = inv[codes.astype(np.int64)].astype(np.uint8)
    assert np.array_equal(vo.dequant_b(codes_p, cb_p), vo.dequant_b(codes, cb))
    cb4 = np.repeat(cb, 4, axis=0)           # four identical codebooks == one codebook
    assert np.array_equal(vo.vq_gemm_b(x, codes, cb4), vo.vq_gemm_b(x, codes, cb))
    assert np.array_equal(vo.vq_gemm_b(x, codes, cb[0]), vo.vq_gemm_b(x, codes, cb))   # [E,v] == [1,E,v]


def test_power_of_two_scaling_is_exact():
    rng = np.random.default_rng(14)
    x, codes, cb = _rand_b(rng, 4, 64, 16, 8, 256, 2, 8)
    y = vo.vq_gemm_b(x, codes, cb)
    y4 = vo.vq_gemm_b((x * np.float16(4)).astype(np.float16), codes, cb)
    assert np.array_equal(y4, (y.astype(np.float32) * 4).astype(np.float16))


def test_geometry_a_equals_explicit_dequant_then_gemm():
    rng = np.random.default_rng(15)
    M, K, Nc = 5, 40, 16
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = rng.integers(0, 256, size=(K, Nc)).astype(np.uint8)
    cb = rng.standard_normal((Nc // 4, 256, 2)).astype(np.float16)
    dec = vo.dequant_a(w, cb)
    assert np.array_equal(vo.vq_gemm_a(x, w, cb), vo.gemm(x, dec))
    assert np.array_equal(c_oracle.vq_gemm_a(x, w, cb), c_oracle.gemm_nn(x, dec))
    e1, _ = vo.rel_err(c_oracle.vq_gemm_a(x, w, cb), vo.vq_gemm_a(x, w, cb, acc=np.float64))
    assert e1 <= 2e-3
    # column 2n+r of the output only depends on code column n: zeroing another column's codes changes nothing there
    w2 = w.copy()
    w2[:, 3] = 0
    y, y2 = vo.vq_gemm_a(x, w, cb), vo.vq_gemm_a(x, w2, cb)
    keep = np.ones(2 * Nc, dtype=bool)
    keep[6:8] = False
    assert np.array_equal(y[:, keep], y2[:, keep])


def test_out_of_range_codes_are_rejected():
    cb = np.zeros((1, 5, 2), dtype=np.float16)
    codes = np.array([[5]], dtype=np.uint8)
    with pytest.raises(ValueError):
        vo.dequant_b(codes, cb)
    with pytest.raises(ValueError):
        c_oracle.dequant_b(codes, cb)


def test_empty_shapes():
    cb = np.zeros((1, 256, 8), dtype=np.float16)
    assert vo.dequant_b(np.zeros((0, 4), dtype=np.uint8), cb).shape == (0, 32)
    y = vo.vq_gemm_b(np.zeros((0, 32), dtype=np.float16), np.zeros((6, 4), dtype=np.uint8), cb)
    assert y.shape == (0, 6)


# ---------------------------------------------------------------- committed fixtures
def _sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.mark.parametrize("name", ["C1", "REF_small"])
def test_golden_fixture(name):
    """Seeded inputs hash to the recorded digests and the oracle reproduces the recorded outputs."""
    from tests.golden.make_golden import FIXTURE_SPECS, fixture_problem
    meta = json.load(open(os.path.join(GOLDEN, f"{name}.json")))
    data = np.load(os.path.join(GOLDEN, f"{name}.npz"))
    spec = FIXTURE_SPECS[name]
    x, codes, cb = fixture_problem(spec)
    assert _sha(x) == meta["sha256"]["x"]
    assert _sha(codes) == meta["sha256"]["codes"]
    assert _sha(cb) == meta["sha256"]["codebook"]
    if spec.geometry == "B":
        w = vo.dequant_b(codes, cb)
        y = vo.vq_gemm_b(x, codes, cb)
        yc = c_oracle.vq_gemm_b(x, codes, cb)
    else:
        w = vo.dequant_a(codes, cb)
        y = vo.vq_gemm_a(x, codes, cb)
        yc = c_oracle.vq_gemm_a(x, codes, cb)
    assert _sha(w) == meta["sha256"]["w_dequant"]
    ri, ci = data["sample_rows"], data["sample_cols"]
    assert np.array_equal(w[data["w_rows"]][:, data["w_cols"]].view(np.uint16), data["w_samples"].view(np.uint16))
    for got in (y, yc):
        e1, _ = vo.rel_err(got[ri][:, ci], data["y_samples_f64"])
        assert e1 <= 2e-3


# ---- nearest-codeword encoder (the quantiser's assignment step) -------------------------------

def _rand_encode_case(rng, N, K, v, E, G):
    w = rng.standard_normal((N, K)).astype(np.float16)
    cb = rng.standard_normal((G, E, v)).astype(np.float16)
    return w, cb


@pytest.mark.parametrize("N,K,v,E,G,bits", [(8, 32, 8, 16, 1, 8), (12, 24, 4, 300, 3, 16), (6, 20, 2, 7, 2, 8)])
def test_encoder_picks_a_nearest_entry(N, K, v, E, G, bits):
    """The C encoder (float32 fma distances) against brute force in float64: the entry it picks
    is a nearest one up to float32 rounding of the distances."""
    rng = np.random.default_rng(7)
    w, cb = _rand_encode_case(rng, N, K, v, E, G)
    codes = c_oracle.encode_b(w, cb, bits)
    assert codes.dtype == (np.uint8 if bits == 8 else np.uint16) and codes.shape == (N, K // v)
    d = vo.encode_b_distances(w, cb)                         # [N,J,E] float64
    picked = np.take_along_axis(d, codes.astype(np.int64)[:, :, None], axis=2)[:, :, 0]
    best = d.min(axis=2)
    assert np.all(picked <= best * (1 + 1e-5) + 1e-12)
    # where the nearest entry is clearly nearest (no near-tie) the index itself is pinned
    second = np.partition(d, 1, axis=2)[:, :, 1]
    clear = second > best * (1 + 1e-4) + 1e-9
    assert clear.mean() > 0.9
    assert np.array_equal(codes[clear], d.argmin(axis=2)[clear].astype(codes.dtype))


def test_encoder_known_answers_and_ties():
    # hand-made: 2-vectors, codebook {(0,0),(1,0),(0,1),(1,0) again}; ties go to the lowest index
    cb = np.array([[[0, 0], [1, 0], [0, 1], [1, 0]]], dtype=np.float16)
    w = np.array([[0.9, 0.1, 0.1, 0.8, 0.5, 0.0, 0.5, 0.5]], dtype=np.float16)
    # (0.9,0.1)->1 (not its duplicate 3); (0.1,0.8)->2; (0.5,0)->tie of 0 and 1 -> 0;
    # (0.5,0.5)-> d=0.5 for entries 0,1,2,3 -> 0
    assert c_oracle.encode_b(w, cb, 8).tolist() == [[1, 2, 0, 0]]
    assert c_oracle.encode_b(w, cb, 16).tolist() == [[1, 2, 0, 0]]


def test_encoder_inverts_the_dequantiser():
    """encode(dequant(codes)) == codes when the entries of a codebook are distinct (distance 0 is
    reached by exactly one entry), per codebook block."""
    rng = np.random.default_rng(11)
    G, E, v, N, K = 2, 64, 4, 16, 32
    cb = rng.standard_normal((G, E, v)).astype(np.float16)
    assert all(len({tuple(e) for e in cb[g].tolist()}) == E for g in range(G))
    codes = rng.integers(0, E, (N, K // v)).astype(np.uint8)
    w = vo.dequant_b(codes, cb)
    assert np.array_equal(c_oracle.encode_b(w, cb, 8), codes)
    # a NaN vector keeps entry 0, whatever the codebook
    w[3, 4:8] = np.nan
    assert c_oracle.encode_b(w, cb, 8)[3, 1] == 0


def test_silu_mul_known_values_and_an_independent_formula():
    a = np.array([[0.0, 20.0, -20.0, 1.0, 3.0, 2.0, 5.0, 4.0]], dtype=np.float16)
    got = vo.silu_mul(a)
    # silu(0) = 0; silu(20) = 20 to fp16 precision; silu(-20) * 5 = -100 / (1 + e^20); silu(1) = 0.731058...
    want = np.array([[0.0, 40.0, -100.0 / (1.0 + np.exp(20.0)), 4.0 / (1.0 + np.exp(-1.0))]]).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    rng = np.random.default_rng(3)
    a = (rng.standard_normal((7, 26)) * 3).astype(np.float16)
    g, u = a[:, :13].astype(np.float64), a[:, 13:].astype(np.float64)
    other = (g * 0.5 * (1.0 + np.tanh(g / 2.0)) * u).astype(np.float16)   # silu(g) = g (1 + tanh(g/2)) / 2
    got = vo.silu_mul(a)
    # the two formulas round differently in the last float64 bit at most: the fp16 results agree
    # except where the product sits on a rounding boundary
    assert np.max(np.abs(got.view(np.int16).astype(np.int32) - other.view(np.int16).astype(np.int32))) <= 1
    assert np.array_equal(vo.silu_mul(np.zeros((2, 6), dtype=np.float16)), np.zeros((2, 3), dtype=np.float16))


def test_additive_stages_side_by_side_along_k_known_answer():
    """The residual mode's identity, pinned by hand: stages laid side by side along K with their
    indices offset into a merged codebook, multiplied against [X, X], give X times the sum of the
    stage weights."""
    # stage 0 entries 0..1, stage 1 entries 2..3 (vectors of two)
    cb = np.array([[1, 2], [3, 4], [10, 20], [30, 40]], dtype=np.float16)
    stage0 = np.array([[0, 1], [1, 1]], dtype=np.uint8)          # W0 rows: [1 2 3 4], [3 4 3 4]
    stage1 = np.array([[1, 0], [0, 0]], dtype=np.uint8) + 2      # W1 rows: [30 40 10 20], [10 20 10 20]
    codes = np.concatenate([stage0, stage1], axis=1)
    x = np.array([[1, 0, 0, 0], [1, 1, 1, 1], [2, -1, 0, 3]], dtype=np.float16)
    # W0 + W1 rows: [31 42 13 24], [13 24 13 24]
    want = np.array([[31, 13], [110, 74], [62 - 42 + 72, 26 - 24 + 72]], dtype=np.float16)
    xx = np.concatenate([x, x], axis=1)
    for fn in (vo.vq_gemm_b, c_oracle.vq_gemm_b):
        assert np.array_equal(fn(xx, codes, cb), want), fn


# ---- packed code layout of the decode kernel -------------------------------------------------
def test_pack_codes_known_answer():
    # 8-vectors, 8-bit codes: 8 codes per lane load, one wave load per 256 k.  16 rows x 32 codes
    # holding code[n][j] = n*32 + j (mod 256): the packed order is k-group, then row, then the lane's
    # 8 codes, so the first 16 pieces are codes 0..7 of rows 0..15, the next 16 codes 8..15, ...
    N, J = 16, 32
    codes = ((np.arange(N)[:, None] * J + np.arange(J)[None, :]) % 256).astype(np.uint8)
    flat = vo.pack_codes_b(codes, 8).reshape(-1)
    assert flat[:8].tolist() == codes[0, :8].tolist()
    assert flat[8:16].tolist() == codes[1, :8].tolist()
    assert flat[15 * 8:16 * 8].tolist() == codes[15, :8].tolist()
    assert flat[16 * 8:17 * 8].tolist() == codes[0, 8:16].tolist()
    assert flat[(3 * 16 + 5) * 8:(3 * 16 + 5) * 8 + 8].tolist() == codes[5, 24:32].tolist()


@pytest.mark.parametrize("N,K,v,bits", [(32, 512, 8, 8), (16, 256, 4, 16), (48, 768, 4, 8), (16, 512, 2, 8),
                                        (32, 256, 2, 16), (16, 1024, 8, 16)])
def test_pack_codes_follows_the_header_formula_element_by_element(N, K, v, bits):
    rng = np.random.default_rng(N + K + v + bits)
    dt = np.uint8 if bits == 8 else np.uint16
    codes = rng.integers(0, 1 << bits, size=(N, K // v)).astype(dt)
    packed = vo.pack_codes_b(codes, v).reshape(-1)
    cpl = (8 if (16 // (bits // 8)) * v * 4 > 256 else 16) // (bits // 8)
    kw = 4 * cpl * v
    i = 0
    for tile in range(N // 16):
        for s in range(K // 256):
            for t in range(256 // kw):
                for q in range(4):
                    for r in range(16):
                        for c in range(cpl):
                            assert packed[i] == codes[tile * 16 + r][(s * 256 + t * kw) // v + q * cpl + c]
                            i += 1
    assert i == packed.size
    assert np.array_equal(vo.pack_codes_b(vo.pack_codes_b(codes, v), v, inverse=True), codes)
    assert sorted(packed.tolist()) == sorted(codes.reshape(-1).tolist())


def test_pack_codes_rejects_shapes_the_kernel_does_not_take():
    with pytest.raises(ValueError):
        vo.pack_codes_b(np.zeros((16, 31), np.uint8), 8)
    with pytest.raises(ValueError):
        vo.pack_codes_b(np.zeros((8, 32), np.uint8), 8)


def test_gated_gemm_is_the_definition_and_agrees_with_the_element_wise_function():
    import math
    rng = np.random.default_rng(11)
    M, K, H, v, E = 3, 16, 32, 4, 16
    cg = rng.integers(0, E, (H, K // v)).astype(np.uint8)
    cu = rng.integers(0, E, (H, K // v)).astype(np.uint8)
    cb = (rng.standard_normal((E, v)) * 0.5).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    bg = rng.standard_normal(H).astype(np.float16)
    bu = rng.standard_normal(H).astype(np.float16)
    codes = vo.interleave_gate_up(cg, cu)
    # the interleave, entry by entry
    assert codes.shape == (2 * H, K // v)
    for o in range(H):
        assert np.array_equal(codes[32 * (o // 16) + o % 16], cg[o]) and np.array_equal(codes[32 * (o // 16) + 16 + o % 16], cu[o])
    bias = vo.interleave_gate_up(bg, bu)
    got = vo.gated_gemm_b(x, codes, cb, bias)
    # the definition as loops over separate gate and up matrices
    wg = vo.dequant_b(cg, cb).astype(np.float64)
    wu = vo.dequant_b(cu, cb).astype(np.float64)
    for m in range(M):
        for o in range(H):
            g = sum(float(x[m, k]) * wg[o, k] for k in range(K)) + float(bg[o])
            u = sum(float(x[m, k]) * wu[o, k] for k in range(K)) + float(bu[o])
            want = np.float16(g / (1.0 + math.exp(-g)) * u)
            assert got[m, o] == want, (m, o, got[m, o], want)
    # with factors that are exact in fp16, the element-wise function on the stacked product gives the same
    xi = rng.integers(-2, 3, (M, K)).astype(np.float16)
    cbi = rng.integers(-2, 3, (E, v)).astype(np.float16)
    pg = (xi.astype(np.float64) @ vo.dequant_b(cg, cbi).astype(np.float64).T).astype(np.float16)
    pu = (xi.astype(np.float64) @ vo.dequant_b(cu, cbi).astype(np.float64).T).astype(np.float16)
    assert np.array_equal(vo.gated_gemm_b(xi, codes, cbi), vo.silu_mul(np.concatenate([pg, pu], axis=1)))
