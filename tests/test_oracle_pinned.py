"""Pins the CPU oracle (oracle/) before anything is compared with it.

Checks are chosen so that a plausible mistake fails one of them: a swapped nibble order fails the
all-words test, a fused multiply-add or a single rounding fails the exact-rational vectors, a
transposed/shifted group index fails the seeded fixture, a wrong rounding rule in compress fails
the packed-equality relation of the fixture.
"""
import hashlib
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN
from golden import make_golden


@pytest.fixture(scope="module")
def seeded():
    packed, scale, bias, t = make_golden.seeded_fixture()
    return packed, scale, bias, t


def test_seeded_fixture_matches_committed_vectors(seeded):
    """The regenerated recipe equals the committed checksums and the committed 16-row slice."""
    packed, scale, bias, t = seeded
    sums = json.load(open(os.path.join(GOLDEN, "seeded_fixture_checksums.json")))
    assert int(packed.astype(np.uint64).sum()) == sums["packed_sum"] == 137407724490
    assert hashlib.sha256(packed.tobytes()).hexdigest() == sums["packed_sha256"]
    assert hashlib.sha256(t.tobytes()).hexdigest() == sums["t_sha256"]
    z = np.load(os.path.join(GOLDEN, "seeded_fixture_rows16.npz"))
    assert np.array_equal(z["packed"], packed[:16]) and np.array_equal(z["t"].view(np.uint16), t[:16].view(np.uint16))


@pytest.mark.parametrize("impl", ["c", "np"])
def test_decompress_seeded_fixture(oracle, seeded, impl):
    """test_numpy relation 1 (test_group_quantize_decompress.py:51): decompress(packed) == t, here bit for bit."""
    packed, scale, bias, t = seeded
    fn = oracle.c_decompress if impl == "c" else oracle.np_decompress
    out = fn(packed, scale, bias)
    assert out.dtype == np.float16 and out.shape == t.shape
    assert np.array_equal(out.view(np.uint16), t.view(np.uint16))


@pytest.mark.parametrize("impl", ["c", "np"])
def test_decompress_committed_slice(oracle, impl):
    z = np.load(os.path.join(GOLDEN, "seeded_fixture_rows16.npz"))
    fn = oracle.c_decompress if impl == "c" else oracle.np_decompress
    out = fn(z["packed"], z["scale"], z["bias"])
    assert np.array_equal(out.view(np.uint16), z["t"].view(np.uint16))


@pytest.mark.parametrize("impl", ["c", "np"])
def test_decompress_all_words_nibble_order(oracle, impl):
    """All 65 536 packed words with scale 1, bias 0: output j of word w is (w >> (12-4j)) & 15,
    evaluated with Python integers (codelet comment group_quantize_decompress_codelet.cpp:11-14)."""
    words = np.arange(65536, dtype=np.uint16).reshape(1, 4096, 16)
    one = np.ones((1, 4096, 1), np.float16)
    zero = np.zeros((1, 4096, 1), np.float16)
    fn = oracle.c_decompress if impl == "c" else oracle.np_decompress
    out = fn(words, one, zero).reshape(65536, 4)
    expect = np.array([[(w >> (12 - 4 * j)) & 15 for j in range(4)] for w in range(65536)], dtype=np.float16)
    assert np.array_equal(out, expect)


@pytest.mark.parametrize("impl", ["c", "np"])
def test_decompress_exact_rational_vectors(oracle, impl):
    """4096 (scale, bias) pairs x 16 codes against exact rational arithmetic with one explicit
    round-to-nearest-even per operation (tests/golden/edge_vectors.npz): subnormals, overflow,
    signed zeros, infinities.  A fused multiply-add fails this on many pairs."""
    z = np.load(os.path.join(GOLDEN, "edge_vectors.npz"))
    n = len(z["scale_bits"])
    # one group of 16 codes 0..15 per pair: words 0x0123 0x4567 0x89ab 0xcdef
    packed = np.tile(np.array([0x0123, 0x4567, 0x89AB, 0xCDEF], np.uint16), (n, 1, 1))
    scale = z["scale_bits"].view(np.float16).reshape(n, 1, 1)
    bias = z["bias_bits"].view(np.float16).reshape(n, 1, 1)
    fn = oracle.c_decompress if impl == "c" else oracle.np_decompress
    with np.errstate(all="ignore"):
        out = fn(packed, scale, bias).view(np.uint16)
    expect = z["expected_bits"]
    nan_e = (expect & 0x7C00 == 0x7C00) & (expect & 0x3FF != 0)
    nan_o = (out & 0x7C00 == 0x7C00) & (out & 0x3FF != 0)
    assert np.array_equal(nan_e, nan_o)
    assert np.array_equal(out[~nan_e], expect[~nan_e])


def test_exact_rational_vectors_would_catch_fma():
    """The committed vectors distinguish two roundings from one (sanity of the pin itself)."""
    z = np.load(os.path.join(GOLDEN, "edge_vectors.npz"))
    s = z["scale_bits"].view(np.float16).astype(np.float64)[:, None]
    b = z["bias_bits"].view(np.float16).astype(np.float64)[:, None]
    with np.errstate(all="ignore"):
        fused = (np.arange(16, dtype=np.float64)[None, :] * s + b).astype(np.float16).view(np.uint16)
    finite = (z["expected_bits"] & 0x7C00) != 0x7C00
    assert (fused[finite] != z["expected_bits"][finite]).mean() > 0.02


def test_decompress_invariants(oracle):
    rng = np.random.default_rng(5)
    packed = rng.integers(0, 65536, (7, 3, 5), dtype=np.uint16)
    scale = rng.normal(0, 1, (7, 3, 1)).astype(np.float16)
    bias = rng.normal(0, 1, (7, 3, 1)).astype(np.float16)
    out0 = oracle.c_decompress(packed, np.zeros_like(scale), bias)
    assert np.array_equal(out0, np.broadcast_to(bias, (7, 3, 20)).reshape(7, 60))
    zero_codes = oracle.c_decompress(np.zeros_like(packed), scale, bias)
    assert np.array_equal(zero_codes, np.broadcast_to(bias, (7, 3, 20)).reshape(7, 60))
    # dim handling equals the reference's pop/insert permutation
    out = oracle.c_decompress(packed, scale, bias)
    assert np.array_equal(oracle.c_decompress(packed, scale, bias, dim=0), out.T)
    assert np.array_equal(oracle.np_decompress(packed, scale, bias, dim=0), out.T)
    assert np.array_equal(oracle.c_decompress(packed, scale, bias, dim=1), out)


def test_c_and_numpy_oracles_agree_on_random_inputs(oracle):
    rng = np.random.default_rng(9)
    packed = rng.integers(0, 65536, (33, 9, 6), dtype=np.uint16)
    scale = (rng.normal(0, 1, (33, 9, 1)) * 10.0 ** rng.integers(-6, 3, (33, 9, 1))).astype(np.float16)
    bias = (rng.normal(0, 1, (33, 9, 1)) * 10.0 ** rng.integers(-6, 3, (33, 9, 1))).astype(np.float16)
    a = oracle.c_decompress(packed, scale, bias).view(np.uint16)
    b = oracle.np_decompress(packed, scale, bias).view(np.uint16)
    assert np.array_equal(a, b)


# ----------------------------------------------------------------------------------- compress


@pytest.mark.parametrize("impl", ["c", "np"])
def test_compress_seeded_fixture(oracle, seeded, impl):
    """test_numpy relations 2-4 (test_group_quantize_decompress.py:52-58)."""
    packed, scale, bias, t = seeded
    fn = oracle.c_compress if impl == "c" else oracle.np_compress
    p, s, b = fn(t, 64)
    assert p.dtype == np.uint16 and p.shape == packed.shape
    assert np.array_equal(p, packed)
    np.testing.assert_allclose(scale.astype(np.float32), s.astype(np.float32), atol=1e-3, rtol=0)
    np.testing.assert_allclose(bias.astype(np.float32), b.astype(np.float32), atol=1e-3, rtol=0)
    assert np.array_equal(b, bias)  # bias = min is exact


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_compress_structure_and_round_trip(oracle, dtype):
    """Config-1 style weight (1024 x 1024 ~ N(0, 0.02), group 64): the arg-min of every group gets
    code 0 and the arg-max code 15, codes stay in [0, 15], pack and unpack are inverses, and the
    round-trip error is within scale/2 plus fp16 rounding slack."""
    rng = np.random.default_rng(0)
    w = rng.normal(0, 0.02, (1024, 1024)).astype(dtype)
    pc, sc, bc = oracle.c_compress(w, 64)
    pn, sn, bn = oracle.np_compress(w, 64)
    assert np.array_equal(pc, pn) and np.array_equal(sc, sn) and np.array_equal(bc, bn)
    codes = np.stack([(pc >> s) & 15 for s in (12, 8, 4, 0)], -1).reshape(1024, 16, 64)
    g = w.reshape(1024, 16, 64)
    assert np.all(np.take_along_axis(codes, g.argmin(-1)[..., None], -1) == 0)
    assert np.all(np.take_along_axis(codes, g.argmax(-1)[..., None], -1) == 15)
    dec = oracle.c_decompress(pc, sc, bc).astype(np.float64).reshape(1024, 16, 64)
    err = np.abs(dec - g.astype(np.float64))
    ulp = np.spacing(np.maximum(np.abs(g).max(-1, keepdims=True), 1e-4).astype(np.float16)).astype(np.float64)
    assert np.all(err <= sc.astype(np.float64) / 2 + 4 * ulp)


def test_compress_dim_and_nonfinite(oracle):
    rng = np.random.default_rng(3)
    w = rng.normal(0, 1, (64, 24)).astype(np.float16)
    p0, s0, b0 = oracle.c_compress(w, 16, dim=0)
    p1, s1, b1 = oracle.c_compress(np.ascontiguousarray(w.T), 16, dim=-1)
    assert np.array_equal(p0, p1) and np.array_equal(s0, s1)
    w[3, 5] = np.inf
    for fn in (oracle.c_compress, oracle.np_compress):
        with pytest.raises(ValueError):
            fn(w, 8)


def test_constant_group_is_defined(oracle):
    w = np.full((2, 32), 0.25, np.float16)
    for fn in (oracle.c_compress, oracle.np_compress):
        p, s, b = fn(w, 16)
        assert not p.any() and not s.any() and np.all(b == np.float16(0.25))
        assert np.array_equal(oracle.c_decompress(p, s, b), w)


# ------------------------------------------------------------------------------------- linear


def test_linear_oracle_is_a_matmul(oracle):
    rng = np.random.default_rng(1)
    x = rng.normal(0, 1, (5, 96)).astype(np.float16)
    w = rng.normal(0, 0.02, (40, 96)).astype(np.float16)
    ob = rng.normal(0, 1, (40,)).astype(np.float16)
    ref = x.astype(np.float64) @ w.astype(np.float64).T + ob.astype(np.float64)
    np.testing.assert_allclose(oracle.c_linear(x, w, ob), ref, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.np_linear(x, w, ob), ref, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(oracle.c_linear(x, w), x.astype(np.float64) @ w.astype(np.float64).T, rtol=1e-6, atol=1e-7)


def test_activation_oracle(oracle):
    """The epilogue restatement against scalar evaluation and against what the functions must
    satisfy: gelu(v) - gelu(-v) = v, gelu(0) = 0, gelu -> identity / 0 far from the origin, and the
    known value of the tanh form at 1 (0.841192 to six places; the erf form gives 0.841345)."""
    import math

    grid = np.linspace(-8, 8, 1601)
    g = oracle.np_activation(grid, "gelu_tanh")
    want = [0.5 * v * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (v + 0.044715 * v * v * v))) for v in grid]
    np.testing.assert_allclose(g, want, rtol=0, atol=1e-15)
    np.testing.assert_allclose(g - g[::-1], grid, atol=1e-12)
    assert oracle.np_activation(np.array([0.0]), "gelu_tanh")[0] == 0.0
    assert abs(oracle.np_activation(np.array([1.0]), "gelu_tanh")[0] - 0.841192) < 5e-7
    assert abs(g[-1] - 8.0) < 1e-9 and abs(g[0]) < 1e-9
    r = oracle.np_activation(grid, "relu")
    assert np.array_equal(r, np.where(grid > 0, grid, 0.0))
    assert oracle.np_activation(grid, None) is grid
    with pytest.raises(ValueError):
        oracle.np_activation(grid, "swish")
