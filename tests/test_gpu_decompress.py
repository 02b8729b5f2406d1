"""GPU parity of the standalone decompress: bit-exact against the oracle, the reference's seeded
fixture and the exact-rational vectors; every call goes through the C ABI (gq_decompress_f16*)."""
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN
from golden import make_golden
from gq_testlib import assert_bits_equal, config2_weight, to_dev
from popxl_addons.ops.group_quantize_decompress import (
    group_quantize_compress_numpy,
    group_quantize_decompress,
)

pytestmark = pytest.mark.gpu


def _run(packed, scale, bias, device, dim=-1):
    out = group_quantize_decompress(to_dev(packed, device), to_dev(scale, device), to_dev(bias, device), dim)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_seeded_fixture_full(hip, device, oracle):
    """The reference's device test (test_group_quantize_decompress.py:71-91, atol 1e-2 there) at
    full size, held to bit-exactness against the fixture's own expected tensor."""
    packed, scale, bias, t = make_golden.seeded_fixture()
    out = _run(packed, scale, bias, device)
    assert_bits_equal(out, t, "seeded fixture")
    np.testing.assert_allclose(t.astype(np.float32), out.astype(np.float32), atol=1e-2, rtol=0)
    out_t = _run(packed, scale, bias, device, dim=0)
    assert_bits_equal(out_t, t.T, "seeded fixture, dim=0")


def test_exact_rational_vectors(hip, device):
    """Subnormal / overflowing / infinite / signed-zero scale and bias: two roundings, no fma,
    denormals kept."""
    z = np.load(os.path.join(GOLDEN, "edge_vectors.npz"))
    n = len(z["scale_bits"])
    packed = np.tile(np.array([0x0123, 0x4567, 0x89AB, 0xCDEF], np.uint16), (n, 1, 1))
    scale = z["scale_bits"].view(np.float16).reshape(n, 1, 1)
    bias = z["bias_bits"].view(np.float16).reshape(n, 1, 1)
    out = _run(packed, scale, bias, device)
    assert_bits_equal(out, z["expected_bits"].view(np.float16), "exact vectors")
    # same pairs through the 2-byte-per-lane kernel (n_ids odd) and the transposed kernel
    packed3 = np.tile(np.array([0x0123, 0x4567, 0x89AB], np.uint16), (n, 1, 1))
    out = _run(packed3, scale, bias, device)
    assert_bits_equal(out, z["expected_bits"].view(np.float16)[:, :12], "exact vectors, scalar kernel")
    out = _run(packed, scale, bias, device, dim=0)
    assert_bits_equal(out, z["expected_bits"].view(np.float16).T, "exact vectors, transposed kernel")


def test_all_65536_words(hip, device, oracle):
    words = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(4)
    for n_ids in (16, 2, 1):
        packed = words.reshape(8, -1, n_ids)
        scale = rng.normal(0, 0.01, (*packed.shape[:2], 1)).astype(np.float16)
        bias = rng.normal(0, 0.1, (*packed.shape[:2], 1)).astype(np.float16)
        assert_bits_equal(_run(packed, scale, bias, device), oracle.c_decompress(packed, scale, bias), f"n_ids={n_ids}")


@pytest.mark.parametrize("rows", [1, 3, 17, 130])
@pytest.mark.parametrize("n_groups", [1, 5])
@pytest.mark.parametrize("n_ids", [1, 2, 3, 4, 6, 8, 16, 32, 40])
def test_ragged_shapes_all_dims(hip, device, oracle, rows, n_groups, n_ids):
    rng = np.random.default_rng(rows * 1000 + n_groups * 100 + n_ids)
    packed = rng.integers(0, 65536, (rows, n_groups, n_ids), dtype=np.uint16)
    scale = rng.normal(0, 0.01, (rows, n_groups, 1)).astype(np.float16)
    bias = rng.normal(0, 0.1, (rows, n_groups, 1)).astype(np.float16)
    want = oracle.c_decompress(packed, scale, bias)
    for dim in (-1, 0, 1):
        got = _run(packed, scale, bias, device, dim)
        assert_bits_equal(got, want.T if dim == 0 else want, f"dim={dim}")
    # rank-2 scale / bias are accepted like the reference wrapper does
    got = _run(packed, scale[..., 0], bias[..., 0], device)
    assert_bits_equal(got, want, "rank-2 scale/bias")


@pytest.mark.parametrize("rows", [8, 136, 200, 256])
@pytest.mark.parametrize("n_groups,n_ids", [(4, 8), (3, 32), (2, 16), (16, 16), (1, 64)])
def test_transposed_tile_kernel(hip, device, oracle, rows, n_groups, n_ids):
    """dim=0 through the 128 x 128 tile kernel (columns a multiple of 128, rows a multiple of 8,
    8 or more uint16 per group): bit-exact, and nothing is written outside the result."""
    rng = np.random.default_rng(rows * 100 + n_groups * 10 + n_ids)
    packed = rng.integers(0, 65536, (rows, n_groups, n_ids), dtype=np.uint16)
    scale = rng.normal(0, 0.01, (rows, n_groups, 1)).astype(np.float16)
    bias = rng.normal(0, 0.1, (rows, n_groups, 1)).astype(np.float16)
    want_t = oracle.c_decompress(packed, scale, bias).T
    assert_bits_equal(_run(packed, scale, bias, device, 0), want_t, "tile kernel")
    p_dev, s_dev, b_dev = to_dev(packed, device), to_dev(scale, device), to_dev(bias, device)
    buf = torch.full((want_t.size + 128,), 123.0, dtype=torch.float16, device=device)
    hip.call("gq_decompress_f16_transposed", p_dev.data_ptr(), s_dev.data_ptr(), b_dev.data_ptr(), buf.data_ptr() + 128,
             rows, n_groups, n_ids, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    res = buf.cpu().numpy()
    assert_bits_equal(res[64 : 64 + want_t.size].reshape(want_t.shape), want_t, "guarded buffer")
    assert np.all(res[:64] == 123.0) and np.all(res[64 + want_t.size :] == 123.0), "wrote out of bounds"


def test_alignment_fallbacks(hip, device, oracle):
    rng = np.random.default_rng(8)
    packed = rng.integers(0, 65536, (67, 9, 16), dtype=np.uint16)
    scale = rng.normal(0, 0.01, (67, 9, 1)).astype(np.float16)
    bias = rng.normal(0, 0.1, (67, 9, 1)).astype(np.float16)
    want = oracle.c_decompress(packed, scale, bias)
    assert_bits_equal(_run(packed, scale, bias, device), want, "aligned")
    # pointers that are only 2-, 4- or 8-byte aligned, and a guarded output buffer
    p_dev, s_dev, b_dev = to_dev(packed, device), to_dev(scale, device), to_dev(bias, device)
    n_out = want.size
    for in_off, out_off in ((1, 0), (2, 0), (4, 0), (0, 1), (0, 4), (3, 5)):
        buf_in = torch.zeros(packed.size + 16, dtype=torch.uint16, device=device)
        buf_in[in_off : in_off + packed.size] = p_dev.reshape(-1)
        buf_out = torch.full((n_out + 64,), 123.0, dtype=torch.float16, device=device)
        hip.call(
            "gq_decompress_f16", buf_in.data_ptr() + 2 * in_off, s_dev.data_ptr(), b_dev.data_ptr(),
            buf_out.data_ptr() + 2 * (16 + out_off), 67, 9, 16, torch.cuda.current_stream().cuda_stream,
        )
        torch.cuda.synchronize()
        res = buf_out.cpu().numpy()
        assert_bits_equal(res[16 + out_off : 16 + out_off + n_out].reshape(want.shape), want, f"offsets {in_off},{out_off}")
        assert np.all(res[: 16 + out_off] == 123.0) and np.all(res[16 + out_off + n_out :] == 123.0), "wrote out of bounds"


def test_config2_full_size(hip, device, oracle):
    """Benchmark configuration 2: 4096 x 16384, group 64, outliers; bit-exact against the numpy
    oracle, plus the size-independent round-trip property compress(decompress(p)) == p."""
    w = config2_weight()
    packed, scale, bias = group_quantize_compress_numpy(w, 64)
    assert packed.shape == (4096, 256, 16)
    got = _run(packed, scale, bias, device)
    want = oracle.np_decompress(packed, scale, bias)
    assert_bits_equal(got, want, "config 2")
    err = np.abs(got.astype(np.float32) - w.astype(np.float32)).reshape(4096, 256, 64)
    assert np.all(err <= scale.astype(np.float32) / 2 + 4 * np.spacing(np.float16(0.16)).astype(np.float32))
    got_t = _run(packed, scale, bias, device, dim=0)
    assert_bits_equal(got_t, want.T, "config 2, dim=0")
