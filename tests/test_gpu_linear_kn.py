"""GPU parity of the fused dequant-matmul for weights grouped along the OUTPUT features
(gq_linear_kn_act_f16: LinearGQ with dim = -1 / 1, the reference's default,
popxl_addons/layers/linear_gq.py:26, 59-62, 99-109) against a float32 matmul over the
oracle-decompressed weight.  Contract: max|y_gpu - y_ref| / max|y_ref| <= 1e-2; regression bound
2e-3 for the whole result and for every output column."""
from functools import partial

import numpy as np
import pytest
import torch

from gq_testlib import activations, assert_bits_equal, normalised_error, to_dev
from popxl_addons.layers.linear_gq import LinearGQ
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy
from popxl_addons.testing_utils import TensorInput, run_module
from test_gpu_fused import assert_close

pytestmark = pytest.mark.gpu


_CASE_WEIGHTS = {}


def _case(oracle, n_out, k_in, gs, m_rows, seed, with_bias, activation=None):
    """Weight [k_in, n_out] grouped along n_out; reference y = act(x @ w_dec + out_bias)."""
    key = (n_out, k_in, gs, seed)  # (large weights take seconds to compress and decompress on the host: once per session)
    if key not in _CASE_WEIGHTS:
        rng = np.random.default_rng(seed)
        w = rng.normal(0, 0.02, (k_in, n_out)).astype(np.float16)
        packed, scale, bias = group_quantize_compress_numpy(w, gs)  # [k_in, n_out / gs, gs / 4]
        out_bias = rng.normal(0, 1, (n_out,)).astype(np.float16)
        w_dec = oracle.np_decompress(packed, scale, bias)  # [k_in, n_out]
        _CASE_WEIGHTS[key] = (packed, scale, bias, out_bias, np.ascontiguousarray(w_dec.T))
    packed, scale, bias, out_bias, w_dec_t = _CASE_WEIGHTS[key]
    x = activations(m_rows, k_in, seed + 1)
    out_bias = out_bias if with_bias else None
    y_ref = oracle.np_linear(x, w_dec_t, out_bias, activation)
    return x, packed, scale, bias, out_bias, y_ref


def _call(hip, x, packed, scale, bias, out_bias, n_out, k_in, gs, device, act=0, workspace=None, packed_offset=0):
    xd, sd, bd = (to_dev(a, device) for a in (x, scale, bias))
    raw = torch.zeros(packed.nbytes + 64, dtype=torch.uint8, device=device)
    raw[packed_offset : packed_offset + packed.nbytes] = torch.from_numpy(packed.view(np.uint8).reshape(-1)).to(device)
    od = None if out_bias is None else to_dev(out_bias, device)
    m_rows = x.shape[0]
    need = hip.load().gq_linear_kn_workspace_bytes(m_rows, n_out, k_in, gs)
    assert need >= 0
    if workspace is None and need > 0:
        workspace = torch.zeros(need, dtype=torch.uint8, device=device)
    y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call("gq_linear_kn_act_f16", xd.data_ptr(), m_rows, raw.data_ptr() + packed_offset, sd.data_ptr(), bd.data_ptr(),
             0 if od is None else od.data_ptr(), y.data_ptr(), n_out, k_in, gs, act,
             0 if workspace is None else workspace.data_ptr(), 0 if workspace is None else workspace.numel(),
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    if workspace is not None and need > 0:
        assert not workspace[:16384].any(), "arrival counters must be back at zero"
    return y.cpu().numpy()


@pytest.mark.parametrize("k_in,n_out", [(4096, 4096), (4096, 16384), (16384, 4096)])
@pytest.mark.parametrize("m_rows", [1, 2, 3, 4, 8, 16])
def test_decode_benchmark_shapes(hip, device, oracle, k_in, n_out, m_rows):
    """The layer shapes of the 6B stack at decode batches, in the default layout."""
    with_bias = m_rows % 2 == 0
    x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 7, with_bias)
    y = _call(hip, x, packed, scale, bias, ob, n_out, k_in, 64, device)
    assert_close(y, y_ref, (k_in, n_out, m_rows))


@pytest.mark.parametrize("m_rows", [17, 128, 300])
def test_prefill_shapes(hip, device, oracle, m_rows):
    for k_in, n_out, gs in ((4096, 4096, 64), (1024, 16384, 64), (320, 416, 32), (64, 96, 32)):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 13, True)
        y = _call(hip, x, packed, scale, bias, ob, n_out, k_in, gs, device)
        assert_close(y, y_ref, (k_in, n_out, gs, m_rows))


@pytest.mark.parametrize("k_in,n_out,m_rows", [(4096, 4096, 17), (4096, 4096, 40), (16384, 4096, 100), (4096, 16384, 32), (4096, 16384, 48)])
def test_mid_batches(hip, device, oracle, k_in, n_out, m_rows):
    """17 to 128 rows on large weights: gq_linear_kn_workspace_bytes asks for a workspace -- the decode
    kernel's where passes of that kernel over 16 rows each are expected to be fastest (17 rows), the
    prefill kernel's own for dividing K over workgroups otherwise (its tiles alone are too few for
    256 compute units here).  Without a workspace (it is optional above 16 rows) the prefill kernel
    runs undivided -- the same result either way."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 23, True)
    lib = hip.load()
    need = lib.gq_linear_kn_workspace_bytes(m_rows, n_out, k_in, 64)
    assert need > 0
    y = _call(hip, x, packed, scale, bias, ob, n_out, k_in, 64, device)
    assert_close(y, y_ref, (k_in, n_out, m_rows))
    xd, pd, sd, bd, od = (to_dev(a, device) for a in (x, packed, scale, bias, ob))
    y2 = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call("gq_linear_kn_act_f16", xd.data_ptr(), m_rows, pd.data_ptr(), sd.data_ptr(), bd.data_ptr(), od.data_ptr(), y2.data_ptr(),
             n_out, k_in, 64, 0, 0, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert_close(y2.cpu().numpy(), y_ref, "without a workspace")


@pytest.mark.parametrize(
    "k_in,n_out,gs,m_rows",
    [
        (128, 256, 16, 4),  # the reference's layer test shape: generic kernel (group 16)
        (1, 32, 32, 1),
        (7, 64, 64, 3),  # fewer input features than one block of four
        (33, 96, 32, 16),  # ragged K slab, three lanes of a strip
        (100, 544, 32, 5),  # a strip and a bit
        (257, 1024, 128, 2),
        (640, 2080, 32, 9),
        (2048, 576, 64, 16),
        (96, 24, 12, 2),  # generic: group 12
        (40, 8, 8, 16),  # generic: n_out < 32
        (50, 128, 64, 40),  # prefill, k_in % 64 != 0: generic
        (5000, 32, 32, 1),  # many K slabs for one strip
        # groups of 64 and whole strips of 256 outputs, every batch size class, ragged K slabs
        (7, 256, 64, 1),
        (1001, 512, 64, 2),
        (333, 768, 64, 4),
        (2050, 256, 64, 7),
        (515, 1280, 64, 13),
    ],
)
def test_edge_shapes(hip, device, oracle, k_in, n_out, gs, m_rows):
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 11, with_bias)
        y = _call(hip, x, packed, scale, bias, ob, n_out, k_in, gs, device)
        assert_close(y, y_ref, (k_in, n_out, gs, m_rows, with_bias))


def test_activation_alignment_and_workspace_reuse(hip, device, oracle):
    """Epilogues in every kernel of this layout; a packed tensor that is only 2-byte aligned runs
    the generic kernel; one workspace serves calls of different shapes one after the other."""
    ws = torch.zeros(16384 + 64 * 16 * 4096 * 4, dtype=torch.uint8, device=device)
    for activation, code in (("relu", 1), ("gelu_tanh", 2)):
        for k_in, n_out, gs, m_rows in ((1024, 2048, 64, 3), (1024, 4096, 64, 16), (512, 64, 64, 1), (256, 512, 64, 64), (48, 40, 20, 2)):
            x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 5, True, activation)
            y = _call(hip, x, packed, scale, bias, ob, n_out, k_in, gs, device, act=code, workspace=ws)
            assert_close(y, y_ref, (activation, k_in, n_out, m_rows))
    x, packed, scale, bias, ob, y_ref = _case(oracle, 512, 384, 64, 4, 9, True)
    y0 = _call(hip, x, packed, scale, bias, ob, 512, 384, 64, device)
    y2 = _call(hip, x, packed, scale, bias, ob, 512, 384, 64, device, packed_offset=2)
    assert_close(y0, y_ref, "aligned")
    assert_close(y2, y_ref, "2-byte aligned")


def test_result_does_not_depend_on_arrival_order(hip, device, oracle):
    """The K slabs are added in a fixed order by whichever workgroup arrives last: repeated calls
    give the same bits."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, 4096, 16384, 64, 4, 21, False)
    first = _call(hip, x, packed, scale, bias, ob, 4096, 16384, 64, device)
    assert_close(first, y_ref)
    for _ in range(5):
        assert_bits_equal(_call(hip, x, packed, scale, bias, ob, 4096, 16384, 64, device), first)


@pytest.mark.parametrize("batch", [(1,), (4,), (3, 5), (64,), (300,)])
@pytest.mark.parametrize("dim", [-1, 1])
def test_linear_gq_default_layout_is_fused(hip, device, oracle, batch, dim, monkeypatch):
    """LinearGQ with the reference's default dim: decode and prefill batches go through
    gq_linear_kn_act_f16 -- no dense matmul, no decompressed weight in memory."""
    torch.manual_seed(1)
    nn_layer = torch.nn.Linear(512, 384, bias=True)
    layer = LinearGQ(384, True, group_size=64, dim=dim)
    x = np.random.default_rng(0).normal(0, 1, (*batch, 512)).astype(np.float16)

    def no_matmul(*a, **k):
        raise AssertionError("dense matmul on the fused path")

    monkeypatch.setattr(torch.Tensor, "__matmul__", no_matmul)
    monkeypatch.setattr(torch, "matmul", no_matmul)
    (y,) = run_module(layer, TensorInput(x), weights=partial(LinearGQ.torch_mapping, nn_layer=nn_layer, dtype=torch.float16, group_size=64, dim=dim))
    assert y.shape == (*batch, 384)
    v = layer.variables
    assert v.weight_compressed.shape == (512, 6, 16)
    w_dec = oracle.np_decompress(v.weight_compressed.data.cpu().numpy(), v.weight_decompression_scale.data.cpu().numpy(),
                                 v.weight_decompression_bias.data.cpu().numpy())
    y_ref = oracle.np_linear(x.reshape(-1, 512), np.ascontiguousarray(w_dec.T), v.bias.data.cpu().numpy()).reshape(*batch, 384)
    assert_close(y, y_ref, batch)


def test_full_size_default_layout_layer(hip, device, oracle):
    """4096 -> 16384 up-projection in the default layout at batch 1 and 128, weights packed on the
    device from float32 (the torch_mapping route), checked against the oracle."""
    torch.manual_seed(3)
    nn_layer = torch.nn.Linear(4096, 16384, bias=True).to(device)
    layer = LinearGQ(16384, True, group_size=64)
    layer.init_variables(4096, torch.float16, device)
    layer.load_weights(LinearGQ.torch_mapping(layer.variables, nn_layer, dtype=torch.float16, group_size=64))
    v = layer.variables
    # the device packer on float32 input agrees with the numpy packer on the same array
    pn, sn, bn = group_quantize_compress_numpy(nn_layer.weight.T.detach().cpu().numpy(), 64)
    assert np.array_equal(v.weight_compressed.data.cpu().numpy(), pn)
    assert_bits_equal(v.weight_decompression_scale.data.cpu().numpy(), sn, "scale")
    w_dec_t = np.ascontiguousarray(oracle.np_decompress(pn, sn, bn).T)
    for m_rows in (1, 128):
        x = activations(m_rows, 4096, 40 + m_rows)
        y = layer(to_dev(x, device)).cpu().numpy()
        assert_close(y, oracle.np_linear(x, w_dec_t, v.bias.data.cpu().numpy()), m_rows)


def test_fused_projections_default_layout(hip, device):
    """LinearGQ.fuse for layers grouped along the output features: the variables stack along the
    group axis, and the fused layer gives the concatenated outputs."""
    torch.manual_seed(2)
    layers = []
    for _ in range(3):
        nn_layer = torch.nn.Linear(512, 384)
        layer = LinearGQ(384, bias=True, group_size=64)
        variables = layer.init_variables(512, torch.float16, device)
        layer.load_weights(LinearGQ.torch_mapping(variables, nn_layer, dtype=torch.float16, group_size=64))
        layers.append(layer)
    fused = LinearGQ.fuse(layers)
    assert fused.out_features == 1152 and fused.variables.weight_compressed.shape == (512, 18, 16)
    for batch in (2, 40):
        x = torch.randn((batch, 512), device=device, dtype=torch.float16)
        want = torch.cat([layer(x) for layer in layers], dim=-1).float().cpu().numpy()
        got = fused(x).float().cpu().numpy()
        assert normalised_error(got, want) <= 2e-3  # (the K slabs of the two problems differ: other summation order)


@pytest.mark.parametrize("dim", [-1, 0])
def test_layers_on_two_streams_do_not_share_scratch(hip, device, dim):
    """LinearGQ.build takes its K-split scratch (arrival counters, partial sums) per (device, stream):
    two layers that run at the same time on different streams give the results they give alone."""
    from popxl_addons import _gq_hip

    torch.manual_seed(5)
    layers, xs, want = [], [], []
    for i in range(2):
        nn_layer = torch.nn.Linear(4096, 4096, bias=False)
        layer = LinearGQ(4096, bias=False, group_size=64, dim=dim)
        variables = layer.init_variables(4096, torch.float16, device)
        layer.load_weights(LinearGQ.torch_mapping(variables, nn_layer, dtype=torch.float16, group_size=64, dim=dim))
        layers.append(layer)
        # (a decode batch for the default layout, 64 rows for dim=0: the shapes whose K is divided through the scratch)
        xs.append(torch.randn((4 if dim == -1 else 64, 4096), device=device, dtype=torch.float16))
        want.append(layer(xs[-1]).clone())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=device) for _ in layers]
    got = [[], []]
    for _ in range(50):
        for i, (layer, stream) in enumerate(zip(layers, streams)):
            with torch.cuda.stream(stream):
                got[i].append(layer(xs[i]))
    torch.cuda.synchronize()
    keys = [k for k in _gq_hip._kn_workspaces if k[1] in {s.cuda_stream for s in streams}]
    assert len(keys) == 2 and _gq_hip._kn_workspaces[keys[0]].data_ptr() != _gq_hip._kn_workspaces[keys[1]].data_ptr()
    for i in range(2):
        for y in got[i]:
            assert torch.equal(y, want[i])
