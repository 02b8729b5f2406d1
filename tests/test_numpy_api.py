"""The shipped numpy pair (popxl_addons.ops.group_quantize_decompress) against the oracle and the
relations of the reference's own tests (tests/integration/ops/test_group_quantize_decompress.py)."""
import os

import numpy as np
import pytest

from conftest import GOLDEN
from golden import make_golden
from popxl_addons.ops.group_quantize_decompress import (
    group_quantize_compress_numpy,
    group_quantize_decompress_numpy,
)


@pytest.fixture(scope="module")
def seeded():
    return make_golden.seeded_fixture()


def test_numpy(seeded):
    """The reference's test_numpy (:45-58), called without `dim` as the reference does."""
    t_packed, group_scale, group_bias, t = seeded
    t_rec = group_quantize_decompress_numpy(t_packed, group_scale, group_bias)
    t_packed_rec, group_scale_rec, group_bias_rec = group_quantize_compress_numpy(t, group_size=64)
    np.testing.assert_allclose(t, t_rec, atol=1e-6, rtol=0)
    np.testing.assert_allclose(t_packed, t_packed_rec, atol=1e-6, rtol=0)
    np.testing.assert_allclose(group_scale, group_scale_rec, atol=1e-3, rtol=0)
    np.testing.assert_allclose(group_bias, group_bias_rec, atol=1e-3, rtol=0)
    # stronger than the reference asks: bit-exact
    assert np.array_equal(t.view(np.uint16), t_rec.view(np.uint16))
    assert t_packed_rec.dtype == np.uint16 and group_scale_rec.dtype == np.float16


def test_compress_is_finite(seeded):
    """The reference's test_compress_is_finite (:61-68)."""
    t = seeded[3].copy()
    t[0][0] = np.nan
    with pytest.raises(ValueError):
        group_quantize_compress_numpy(t, group_size=64)
    t[0][0] = np.inf
    with pytest.raises(ValueError):
        group_quantize_compress_numpy(t, group_size=64, dim=-1)


def test_decompress_equals_oracle_on_exact_vectors(oracle):
    z = np.load(os.path.join(GOLDEN, "edge_vectors.npz"))
    n = len(z["scale_bits"])
    packed = np.tile(np.array([0x0123, 0x4567, 0x89AB, 0xCDEF], np.uint16), (n, 1, 1))
    scale = z["scale_bits"].view(np.float16).reshape(n, 1, 1)
    bias = z["bias_bits"].view(np.float16).reshape(n, 1, 1)
    with np.errstate(all="ignore"):
        out = group_quantize_decompress_numpy(packed, scale, bias).view(np.uint16)
    expect = z["expected_bits"]
    nan = (expect & 0x7C00 == 0x7C00) & (expect & 0x3FF != 0)
    assert np.array_equal(out[~nan], expect[~nan])
    assert np.all((out[nan] & 0x7C00 == 0x7C00) & (out[nan] & 0x3FF != 0))


@pytest.mark.parametrize("shape", [(5, 3, 1), (2, 7, 4, 16), (4, 8), (1, 1, 1)])
@pytest.mark.parametrize("dim", [-1, 0, 1])
def test_decompress_shapes_and_dim(oracle, shape, dim):
    if dim >= len(shape) - 1 + 1:
        pytest.skip("dim outside the output rank")
    rng = np.random.default_rng(sum(shape))
    packed = rng.integers(0, 65536, shape, dtype=np.uint16)
    scale = rng.normal(0, 0.01, (*shape[:-1], 1)).astype(np.float16)
    bias = rng.normal(0, 0.1, (*shape[:-1], 1)).astype(np.float16)
    got = group_quantize_decompress_numpy(packed, scale, bias, dim)
    want = oracle.c_decompress(packed, scale, bias, dim)
    assert got.shape == want.shape and np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("group_size", [4, 16, 64, 128])
@pytest.mark.parametrize("dim", [-1, 0])
def test_compress_equals_oracle(oracle, dtype, group_size, dim):
    rng = np.random.default_rng(group_size)
    w = rng.normal(0, 0.02, (256, 384)).astype(dtype)
    w[rng.random(w.shape) < 1e-3] *= 8  # outliers
    got = group_quantize_compress_numpy(w, group_size, dim)
    want = oracle.c_compress(w, group_size, dim)
    for g, e in zip(got, want):
        assert g.dtype == e.dtype and g.shape == e.shape and np.array_equal(g.view(np.uint16), e.view(np.uint16))


def test_config1_round_trip(oracle):
    """Benchmark configuration 1: 1024 x 1024 ~ N(0, 0.02), group 64; |error| <= scale/2 (+ fp16 slack)."""
    rng = np.random.default_rng(1)
    w = rng.normal(0, 0.02, (1024, 1024)).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, 64)
    assert packed.shape == (1024, 16, 16) and scale.shape == (1024, 16, 1) and bias.shape == (1024, 16, 1)
    dec = group_quantize_decompress_numpy(packed, scale, bias)
    g = w.reshape(1024, 16, 64).astype(np.float64)
    err = np.abs(dec.reshape(1024, 16, 64).astype(np.float64) - g)
    ulp = np.spacing(np.abs(w.reshape(1024, 16, 64)).max(-1, keepdims=True)).astype(np.float64)
    assert np.all(err <= scale.astype(np.float64) / 2 + 4 * ulp)
    assert np.array_equal(dec, oracle.c_decompress(packed, scale, bias))


def test_constant_group_and_bad_group_size():
    w = np.full((3, 16), -1.5, np.float16)
    p, s, b = group_quantize_compress_numpy(w, 8)
    assert not p.any() and not s.any()
    assert np.array_equal(group_quantize_decompress_numpy(p, s, b), w)
    with pytest.raises(ValueError):
        group_quantize_compress_numpy(w, 6)
    with pytest.raises(ValueError):
        group_quantize_compress_numpy(w, 12)
