"""GPU parity of the fused dequant-GEMV / GEMM entry points (C ABI: gq_gemv_f16, gq_gemm_f16,
gq_linear_f16) against a float32 matmul over the oracle-decompressed weight.
Tolerance: max|y_gpu - y_ref| / max|y_ref| <= 1e-2."""
import numpy as np
import pytest
import torch

from gq_testlib import activations, normal_weight, normalised_error, to_dev
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _call(hip, entry, x, packed, scale, bias, out_bias, n_out, k_in, gs, device):
    xd, pd, sd, bd = (to_dev(a, device) for a in (x, packed, scale, bias))
    od = None if out_bias is None else to_dev(out_bias, device)
    y = torch.full((x.shape[0], n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call(
        entry, xd.data_ptr(), x.shape[0], pd.data_ptr(), sd.data_ptr(), bd.data_ptr(),
        0 if od is None else od.data_ptr(), y.data_ptr(), n_out, k_in, gs, torch.cuda.current_stream().cuda_stream,
    )
    torch.cuda.synchronize()
    return y.cpu().numpy()


def _case(oracle, n_out, k_in, gs, m_rows, seed, with_bias):
    w = normal_weight(n_out, k_in, seed)
    packed, scale, bias = group_quantize_compress_numpy(w, gs)
    x = activations(m_rows, k_in, seed + 1)
    out_bias = np.random.default_rng(seed + 2).normal(0, 1, (n_out,)).astype(np.float16) if with_bias else None
    w_dec = oracle.np_decompress(packed, scale, bias)
    y_ref = oracle.np_linear(x, w_dec, out_bias)
    return x, packed, scale, bias, out_bias, y_ref


@pytest.mark.parametrize("n_out,k_in", [(4096, 4096), (16384, 4096), (4096, 16384)])
@pytest.mark.parametrize("m_rows", [1, 4, 8, 16])
def test_gemv_benchmark_shapes(hip, device, oracle, n_out, k_in, m_rows):
    """Benchmark configurations 3 and 5: decode batches on the layer shapes of the 6B stack."""
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 7, with_bias)
        y = _call(hip, "gq_gemv_f16", x, packed, scale, bias, ob, n_out, k_in, 64, device)
        assert np.isfinite(y).all()
        assert normalised_error(y, y_ref) <= TOL


@pytest.mark.parametrize(
    "n_out,k_in,gs,m_rows",
    [
        (256, 128, 16, 4),  # the reference's layer test shape (generic kernel: group 16)
        (16, 128, 32, 1),
        (17, 256, 64, 3),  # n_out not a multiple of 16
        (100, 384, 128, 16),  # k_in = 3 slots of 128
        (33, 640, 64, 5),
        (48, 1152, 32, 2),  # more chunks than fit one pass of a workgroup? no: ragged last chunk
        (8, 96, 8, 2),  # generic: k_in % 128 != 0
        (5, 12, 12, 16),  # generic: group 12
        (64, 8192, 256, 7),
    ],
)
def test_gemv_edge_shapes(hip, device, oracle, n_out, k_in, gs, m_rows):
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 11, with_bias)
        for entry in ("gq_gemv_f16", "gq_linear_f16"):
            y = _call(hip, entry, x, packed, scale, bias, ob, n_out, k_in, gs, device)
            assert np.isfinite(y).all()
            assert normalised_error(y, y_ref) <= TOL, (entry, with_bias)


def test_gemv_generic_kernel_matches_fast_kernel(hip, device, oracle):
    x, packed, scale, bias, ob, y_ref = _case(oracle, 512, 1024, 64, 8, 3, True)
    try:
        hip.set_option("gemv_variant", 1)
        y_generic = _call(hip, "gq_gemv_f16", x, packed, scale, bias, ob, 512, 1024, 64, device)
    finally:
        hip.set_option("gemv_variant", 0)
    y_fast = _call(hip, "gq_gemv_f16", x, packed, scale, bias, ob, 512, 1024, 64, device)
    assert normalised_error(y_generic, y_ref) <= TOL and normalised_error(y_fast, y_ref) <= TOL
    assert normalised_error(y_fast, y_generic) <= 2e-3


@pytest.mark.parametrize("m_rows", [128, 512, 2048])
def test_gemm_benchmark_shapes(hip, device, oracle, m_rows):
    """Benchmark configuration 4: prefill batches on the [16384 x 4096] weight."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, 16384, 4096, 64, m_rows, 21, m_rows == 512)
    y = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, 16384, 4096, 64, device)
    assert np.isfinite(y).all()
    assert normalised_error(y, y_ref) <= TOL


@pytest.mark.parametrize(
    "n_out,k_in,gs,m_rows",
    [
        (256, 128, 16, 40),  # generic fallback (group 16)
        (128, 64, 64, 17),
        (200, 192, 32, 100),  # ragged m and n tiles
        (130, 320, 64, 129),
        (512, 1024, 128, 256),
        (64, 256, 256, 33),
        (24, 40, 20, 18),  # generic fallback
    ],
)
def test_gemm_edge_shapes(hip, device, oracle, n_out, k_in, gs, m_rows):
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 31, with_bias)
        for entry in ("gq_gemm_f16", "gq_linear_f16"):
            y = _call(hip, entry, x, packed, scale, bias, ob, n_out, k_in, gs, device)
            assert np.isfinite(y).all()
            assert normalised_error(y, y_ref) <= TOL, (entry, with_bias)


@pytest.mark.parametrize("variant", [1, 2, 30, 31, 32, 33, 34])
def test_gemm_every_kernel_shape(hip, device, oracle, variant):
    """Each tile shape of the pipelined kernel (30..34), the LDS-staged tile kernel (2) and the
    generic kernel (1) on ragged problems, including a weight with an odd number of groups per row
    (which the pipelined kernel hands to the tile kernel)."""
    try:
        hip.set_option("gemm_variant", variant)
        for n_out, k_in, gs, m_rows in ((300, 1024, 64, 260), (130, 448, 32, 70), (96, 192, 64, 33)):
            x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 41, True)
            y = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, n_out, k_in, gs, device)
            assert np.isfinite(y).all()
            assert normalised_error(y, y_ref) <= TOL, (variant, n_out, k_in, gs, m_rows)
    finally:
        hip.set_option("gemm_variant", 0)


def test_linearity_at_full_size(hip, device):
    """Size-independent property on the largest shape: y(x1 + x2) = y(x1) + y(x2) for a weight that
    is never decompressed on the host (16384 x 4096, batch 2048 and batch 1)."""
    rng = np.random.default_rng(5)
    n_out, k_in, gs = 16384, 4096, 64
    pd = torch.from_numpy(rng.integers(0, 65536, (n_out, k_in // gs, gs // 4), dtype=np.uint16)).to(device)
    sd = torch.from_numpy(rng.uniform(0.001, 0.004, (n_out, k_in // gs, 1)).astype(np.float16)).to(device)
    bd = torch.from_numpy(rng.normal(-0.03, 0.005, (n_out, k_in // gs, 1)).astype(np.float16)).to(device)
    for m_rows, entry in ((2048, "gq_gemm_f16"), (1, "gq_gemv_f16")):
        x1 = torch.from_numpy(activations(m_rows, k_in, 1)).to(device)
        x2 = torch.from_numpy(activations(m_rows, k_in, 2)).to(device)
        ys = []
        for xd in (x1, x2, x1 + x2):
            y = torch.empty((m_rows, n_out), dtype=torch.float16, device=device)
            hip.call(entry, xd.data_ptr(), m_rows, pd.data_ptr(), sd.data_ptr(), bd.data_ptr(), 0, y.data_ptr(),
                     n_out, k_in, gs, torch.cuda.current_stream().cuda_stream)
            ys.append(y.float())
        torch.cuda.synchronize()
        err = (ys[2] - ys[0] - ys[1]).abs().max().item() / ys[2].abs().max().item()
        assert err <= TOL, (entry, err)
