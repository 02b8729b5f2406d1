"""The reference's layer test (tests/integration/layers/test_linear_gq.py:33-70) on the GPU layer,
and device-side compress parity."""
from functools import partial

import numpy as np
import pytest
import torch

from gq_testlib import assert_bits_equal, config2_weight, normalised_error, to_dev
from popxl_addons.layers.linear_gq import LinearGQ
from popxl_addons.ops.group_quantize_decompress import (
    group_quantize_compress,
    group_quantize_compress_numpy,
    group_quantize_decompress_numpy,
)
from popxl_addons.testing_utils import TensorInput, run_module

pytestmark = pytest.mark.gpu


class LinearGQTorch(torch.nn.Linear):
    """fp32 nn.Linear whose weight is decompress(compress(W)): the reference test's oracle (:18-30)."""

    def __init__(self, group_size, dim, *args, **kwargs):
        super().__init__(*args, **kwargs)
        w = group_quantize_decompress_numpy(
            *group_quantize_compress_numpy(self.weight.T.detach().numpy(), group_size, dim=dim), dim=dim
        )
        self.weight = torch.nn.Parameter(torch.from_numpy(np.ascontiguousarray(w)).T.to(self.bias.dtype).contiguous())


@pytest.mark.parametrize("dim", [0, -1])
@pytest.mark.parametrize("bias", [True, False])
def test_linear_gq(hip, device, dim, bias):
    in_features, out_features, group_size, batch_size = 128, 256, 16, 4
    np.random.seed(0)
    torch.manual_seed(0)
    input = np.random.rand(batch_size, in_features).astype(np.float16)
    torch_layer = LinearGQTorch(group_size=group_size, in_features=in_features, out_features=out_features, bias=True, dim=dim)
    if not bias:
        torch.nn.init.zeros_(torch_layer.bias)
    torch_output = torch_layer(torch.from_numpy(input).to(torch.float)).detach().numpy()

    gq_layer = LinearGQ(out_features, bias, group_size=group_size, dim=dim)
    (gq_out,) = run_module(
        gq_layer,
        TensorInput(input),
        weights=partial(LinearGQ.torch_mapping, nn_layer=torch_layer, dtype=torch.float16, group_size=group_size, dim=dim),
    )
    assert gq_out.dtype == np.float16 and gq_out.shape == (batch_size, out_features)
    np.testing.assert_allclose(gq_out, torch_output.astype(np.float16), atol=0.1)  # the reference's bar (:70)
    assert normalised_error(gq_out, torch_output) <= 1e-2  # the tighter bar of the fused kernels


@pytest.mark.parametrize("batch", [(1,), (8,), (3, 5), (64,), (300,)])
def test_linear_gq_dim0_dispatch_and_leading_dims(hip, device, oracle, batch):
    """dim=0 with group 64: GEMV kernel up to 16 rows, GEMM kernel above; leading dims are kept."""
    torch.manual_seed(1)
    nn_layer = torch.nn.Linear(512, 384, bias=True)
    layer = LinearGQ(384, True, group_size=64, dim=0)
    x = np.random.default_rng(0).normal(0, 1, (*batch, 512)).astype(np.float16)
    (y,) = run_module(layer, TensorInput(x), weights=partial(LinearGQ.torch_mapping, nn_layer=nn_layer, dtype=torch.float16, group_size=64, dim=0))
    assert y.shape == (*batch, 384)
    v = layer.variables
    w_dec = oracle.np_decompress(v.weight_compressed.data.cpu().numpy(), v.weight_decompression_scale.data.cpu().numpy(),
                                 v.weight_decompression_bias.data.cpu().numpy())
    y_ref = oracle.np_linear(x.reshape(-1, 512), w_dec, v.bias.data.cpu().numpy()).reshape(*batch, 384)
    assert normalised_error(y, y_ref) <= 1e-2


@pytest.mark.parametrize("group_size", [8, 16, 32, 64, 128, 256, 512, 12, 40])
def test_device_compress_bit_exact(hip, device, oracle, group_size):
    rng = np.random.default_rng(group_size)
    cols = group_size * 7
    w = rng.normal(0, 0.02, (129, cols)).astype(np.float16)
    w[rng.random(w.shape) < 1e-2] *= 8
    w[5, :group_size] = 0.125  # a constant group
    w[6, : 2 * group_size] = 0.0
    p, s, b = group_quantize_compress(to_dev(w, device), group_size)
    torch.cuda.synchronize()
    pw, sw, bw = oracle.c_compress(w, group_size)
    assert np.array_equal(p.cpu().numpy(), pw)
    assert_bits_equal(s.cpu().numpy(), sw, "scale")
    assert_bits_equal(b.cpu().numpy(), bw, "bias")


def test_device_compress_config2_and_nonfinite(hip, device, oracle):
    w = config2_weight(1024, 16384, seed=4)
    p, s, b = group_quantize_compress(to_dev(w, device), 64)
    pn, sn, bn = group_quantize_compress_numpy(w, 64)
    assert np.array_equal(p.cpu().numpy(), pn)
    assert_bits_equal(s.cpu().numpy(), sn, "scale")
    assert_bits_equal(b.cpu().numpy(), bn, "bias")
    # dim=0 groups along rows
    p0, s0, b0 = group_quantize_compress(to_dev(w[:, :256], device), 64, dim=0)
    pn0, sn0, bn0 = group_quantize_compress_numpy(w[:, :256], 64, dim=0)
    assert np.array_equal(p0.cpu().numpy(), pn0) and np.array_equal(s0.cpu().numpy(), sn0)
    w[7, 9] = np.nan
    with pytest.raises(ValueError):
        group_quantize_compress(to_dev(w, device), 64)
