"""gq_linear_p_act_f16: the fused matmul for weights grouped along the input features (LinearGQ with
dim=0) when the caller also holds the derived copy in the streaming layout (gq_gemv_prepack_f16).
The one-shot GEMV kernel and the pipelined GEMM kernel then read the copy; the arithmetic is that of
gq_linear_act_ws_f16 on the three variables, so the results are the oracle's to the tolerance of the
fused paths AND equal to that entry point's bit for bit."""
import numpy as np
import pytest
import torch

from gq_testlib import activations, assert_bits_equal, normal_weight, to_dev
from popxl_addons._gq_hip import GQ_ERR_MISALIGNED, GQ_ERR_NULL_POINTER, GQ_ERR_UNSUPPORTED, GQHipError
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy
from test_gpu_fused import assert_close

pytestmark = pytest.mark.gpu

_WEIGHTS = {}


def _weight(hip, device, oracle, n_out, k_in, seed):
    key = (n_out, k_in, seed)
    if key not in _WEIGHTS:
        packed, scale, bias = group_quantize_compress_numpy(normal_weight(n_out, k_in, seed), 64)
        dev = tuple(to_dev(a, device) for a in (packed, scale, bias))
        _WEIGHTS[key] = (dev, hip.prepack_gemv(*dev), oracle.np_decompress(packed, scale, bias))
    return _WEIGHTS[key]


def _run(hip, device, x, dev, blob, out_bias, n_out, k_in, act, workspace=None):
    xd = to_dev(x, device)
    od = None if out_bias is None else to_dev(out_bias, device)
    y = torch.full((x.shape[0], n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call("gq_linear_p_act_f16", xd.data_ptr(), x.shape[0], dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
             0 if blob is None else blob.data_ptr(), 0 if od is None else od.data_ptr(), y.data_ptr(), n_out, k_in, 64, act,
             0 if workspace is None else workspace.data_ptr(), 0 if workspace is None else workspace.numel(),
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("m_rows", [128, 384, 512, 2048])
def test_benchmark_prefill_batches(hip, device, oracle, m_rows):
    """Benchmark configuration 4 on the derived copy: every tile shape of the pipelined kernel (128 x 64, 128 x 256
    -- at 384 rows from the variables too, at 512 rows from the copy only --, 256 x 128, 256 x 256)."""
    n_out, k_in = 16384, 4096
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 21)
    x = activations(m_rows, k_in, 22)
    ob = np.random.default_rng(23).normal(0, 1, (n_out,)).astype(np.float16) if m_rows == 512 else None
    y = _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, 0)
    assert_close(y, oracle.np_linear(x, w_dec, ob), m_rows)
    assert_bits_equal(y, _run(hip, device, x, dev, None, ob, n_out, k_in, 0), "against the variables")


@pytest.mark.parametrize("n_out,k_in", [(4096, 4096), (16384, 4096), (4096, 16384), (28672, 4096), (1000, 1536), (16, 512)])
@pytest.mark.parametrize("m_rows", [1, 3, 4, 8, 16])
def test_decode_batches(hip, device, oracle, n_out, k_in, m_rows):
    """Up to 16 rows the GEMV kernels read the copy (every load 1 KiB contiguous, read once): the oracle's result,
    and the bits of the same call on the variables (the same kernel runs on either)."""
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 41)
    x = activations(m_rows, k_in, 42 + m_rows)
    ob = np.random.default_rng(43).normal(0, 1, (n_out,)).astype(np.float16) if m_rows % 2 else None
    y = _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, 1)
    assert_close(y, oracle.np_linear(x, w_dec, ob, "relu"), (n_out, k_in, m_rows))
    assert_bits_equal(y, _run(hip, device, x, dev, None, ob, n_out, k_in, 1), "against the variables")


@pytest.mark.parametrize("n_out,k_in", [(28672, 4096), (28712, 1024), (32768, 512), (3400, 1536)])
@pytest.mark.parametrize("m_rows", [3, 4, 5, 6, 7, 8])
def test_three_to_eight_rows_on_wide_weights(hip, device, oracle, n_out, k_in, m_rows):
    """Weights whose rows alone fill the compute units, k_in <= 4096: the kernel whose waves share the batch rows'
    x (4 x 4 or 2 x 8 (group, batch row) combinations per accumulator; batch rows that do not fill them; a last
    group of row blocks with waves that have no rows, a last row block with 8 rows).  3400 x 1536 stays with
    the other kernels.  The oracle's result from the copy and from the variables, the same bits from both."""
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 41 if n_out == 28672 else 61)
    x = activations(m_rows, k_in, 62 + m_rows)
    ob = np.random.default_rng(63).normal(0, 1, (n_out,)).astype(np.float16) if m_rows % 2 else None
    act, name = ((2, "gelu_tanh") if m_rows == 6 else (0, None))
    y = _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, act)
    assert_close(y, oracle.np_linear(x, w_dec, ob, name), (n_out, k_in, m_rows))
    assert_bits_equal(y, _run(hip, device, x, dev, None, ob, n_out, k_in, act), "against the variables")
    only_copy = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    xd, od = to_dev(x, device), None if ob is None else to_dev(ob, device)
    hip.call("gq_linear_p_act_f16", xd.data_ptr(), m_rows, 0, 0, 0, copy.blob.data_ptr(), 0 if od is None else od.data_ptr(),
             only_copy.data_ptr(), n_out, k_in, 64, act, 0, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert_bits_equal(only_copy.cpu().numpy(), y, "the copy alone")


@pytest.mark.parametrize("n_out,k_in,m_rows", [(4096, 4096, 300), (4096, 16384, 128), (4104, 512, 300), (8200, 1024, 777),
                                               (4104, 1536, 2060), (1000, 4096, 40), (72, 512, 33), (16384, 4096, 64),
                                               (4096, 4096, 17), (4096, 4096, 8)])
def test_shapes_with_and_without_workspace(hip, device, oracle, n_out, k_in, m_rows):
    """Ragged tiles and row blocks (n_out not a multiple of 16: the copy pads the last block), K divided
    over workgroups through the workspace, the 64 x 64 tiles, batches that run as passes of the GEMV
    kernel or as one GEMV, an activation."""
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 31)
    x = activations(m_rows, k_in, 32)
    ob = np.random.default_rng(33).normal(0, 1, (n_out,)).astype(np.float16)
    need = hip.load().gq_gemm_workspace_bytes(m_rows, n_out, k_in, 64)
    ws = torch.zeros(max(need, 16384), dtype=torch.uint8, device=device)
    y_ref = oracle.np_linear(x, w_dec, ob, "gelu_tanh")
    for workspace in (None, ws):
        y = _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, 2, workspace)
        assert_close(y, y_ref, (n_out, k_in, m_rows, workspace is not None))
        assert_bits_equal(y, _run(hip, device, x, dev, None, ob, n_out, k_in, 2, workspace), "against the variables")
        assert not ws[:16384].any(), "arrival counters must be back at zero"


@pytest.mark.parametrize("n_out,k_in,m_rows", [(4096, 4096, 1), (4096, 16384, 8), (28672, 4096, 2), (1000, 1536, 16), (4096, 4096, 40),
                                               (4096, 16384, 128), (4104, 1536, 2060), (16384, 4096, 512)])
def test_the_copy_alone(hip, device, oracle, n_out, k_in, m_rows):
    """packed, scale and bias NULL: a caller that keeps only the copy.  Every kernel reads the copy (one GEMV,
    passes of the GEMV kernel, the GEMM kernel with and without K divided over workgroups): the bits of the
    call that also hands over the variables."""
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 41 if n_out in (28672, 1000) else 31)  # (weights other tests made)
    x = activations(m_rows, k_in, 52)
    ob = np.random.default_rng(53).normal(0, 1, (n_out,)).astype(np.float16)
    need = hip.load().gq_gemm_workspace_bytes(m_rows, n_out, k_in, 64)
    ws = torch.zeros(max(need, 16384), dtype=torch.uint8, device=device)
    for workspace in (None, ws):
        xd, od = to_dev(x, device), to_dev(ob, device)
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        hip.call("gq_linear_p_act_f16", xd.data_ptr(), m_rows, 0, 0, 0, copy.blob.data_ptr(), od.data_ptr(), y.data_ptr(), n_out, k_in,
                 64, 0, 0 if workspace is None else workspace.data_ptr(), 0 if workspace is None else workspace.numel(),
                 torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec, ob), (n_out, k_in, m_rows))
        assert_bits_equal(y.cpu().numpy(), _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, 0, workspace), "with the variables")


@pytest.mark.parametrize("n_out,k_in", [(4096, 4096), (28672, 4096), (4096, 16384), (1000, 1536)])
@pytest.mark.parametrize("m_rows", [1, 2, 4, 8, 16])
def test_rows_of_x_a_stride_apart(hip, device, oracle, n_out, k_in, m_rows):
    """gq_linear_p_strided_f16: x as a column slice of a wider matrix (rows 16-byte aligned: every kernel of the
    decode batches reads it where it lies) gives the bits of the call on the gathered x, from the copy, from the
    variables and from the copy alone; a slice whose rows are NOT 16-byte aligned runs the kernels for a
    misaligned x on the variables (the oracle's result)."""
    dev, copy, w_dec = _weight(hip, device, oracle, n_out, k_in, 41 if n_out in (28672, 1000) or k_in == 16384 else 31)
    wide = activations(m_rows, k_in + 200, 72 + m_rows)
    wd = to_dev(wide, device)
    ob = np.random.default_rng(73).normal(0, 1, (n_out,)).astype(np.float16)
    od = to_dev(ob, device)
    stream = torch.cuda.current_stream().cuda_stream

    def strided(offset, variables, blob):
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        v = [t.data_ptr() for t in dev] if variables else [0, 0, 0]
        hip.call("gq_linear_p_strided_f16", wd.data_ptr() + 2 * offset, k_in + 200, m_rows, *v, copy.blob.data_ptr() if blob else 0,
                 od.data_ptr(), y.data_ptr(), n_out, k_in, 64, 1, stream)
        torch.cuda.synchronize()
        return y.cpu().numpy()

    for offset in (0, 136):
        x = np.ascontiguousarray(wide[:, offset : offset + k_in])
        gathered = _run(hip, device, x, dev, copy.blob, ob, n_out, k_in, 1)
        assert_close(gathered, oracle.np_linear(x, w_dec, ob, "relu"), (n_out, k_in, m_rows, offset))
        for variables, blob in ((True, True), (True, False), (False, True)):
            assert_bits_equal(strided(offset, variables, blob), gathered, (offset, variables, blob))
    x = np.ascontiguousarray(wide[:, 3 : 3 + k_in])
    assert_close(strided(3, True, True), oracle.np_linear(x, w_dec, ob, "relu"), "rows of x not 16-byte aligned")
    with pytest.raises(GQHipError) as e:
        strided(3, False, True)
    assert e.value.code == GQ_ERR_MISALIGNED


@pytest.mark.parametrize("seed", range(24))
def test_random_decode_problems_through_every_route(hip, device, oracle, seed):
    """Seeded random problems at decode batches: shapes that fill or do not fill chunks of 512 features and groups of
    8 row blocks, group sizes 32 / 64 / 128, one to sixteen rows, x gathered or a column slice (aligned or not), with
    the copy (where one exists), without it, and the copy alone: whichever kernel the routing picks, the oracle's
    result; the copy and the variables agree bit for bit wherever both run the same kernel (an aligned x)."""
    rng = np.random.default_rng(1000 + seed)
    gs = int(rng.choice([32, 64, 64, 64, 128]))
    k_in = int(rng.choice([128, 256, 512, 640, 1024, 1536, 2048, 4096])) if seed % 3 else int(rng.choice([512, 1024, 2048]))
    k_in = max(k_in, gs)
    n_out = int(rng.choice([16, 40, 128, 1000, 3336, 4096])) if seed % 3 else int(rng.choice([26624, 28680, 33000]))
    m_rows = int(rng.integers(1, 17))
    offset = int(rng.choice([0, 0, 8, 24, 3]))
    pad = int(rng.choice([0, 64, 200]))
    w = (rng.normal(0, 0.02, (n_out, k_in)) * np.exp(rng.normal(0, 0.5, (n_out, 1)))).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, gs)
    w_dec = oracle.np_decompress(packed, scale, bias)
    dev = tuple(to_dev(a, device) for a in (packed, scale, bias))
    has_copy = gs == 64 and k_in % 512 == 0
    copy = hip.prepack_gemv(*dev) if has_copy else None
    wide = activations(m_rows, k_in + offset + pad, 2000 + seed)
    x = np.ascontiguousarray(wide[:, offset : offset + k_in])
    ob = rng.normal(0, 1, (n_out,)).astype(np.float16) if seed % 2 else None
    act, name = [(0, None), (1, "relu"), (2, "gelu_tanh")][seed % 3]
    ref = oracle.np_linear(x, w_dec, ob, name)
    wd, od = to_dev(wide, device), None if ob is None else to_dev(ob, device)
    stream = torch.cuda.current_stream().cuda_stream
    aligned = offset % 8 == 0 and (k_in + offset + pad) % 8 == 0

    def strided(variables, blob):
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        v = [t.data_ptr() for t in dev] if variables else [0, 0, 0]
        hip.call("gq_linear_p_strided_f16", wd.data_ptr() + 2 * offset, k_in + offset + pad, m_rows, *v,
                 copy.blob.data_ptr() if blob else 0, 0 if od is None else od.data_ptr(), y.data_ptr(), n_out, k_in, gs, act, stream)
        torch.cuda.synchronize()
        return y.cpu().numpy()

    what = (seed, gs, n_out, k_in, m_rows, offset, pad)
    from_variables = strided(True, False)
    assert_close(from_variables, ref, what)
    assert_close(_run(hip, device, x, dev, None, ob, n_out, k_in, act) if gs == 64 else from_variables, ref, what)
    if has_copy:
        with_copy = strided(True, True)
        assert_close(with_copy, ref, what)
        if aligned:
            assert_bits_equal(with_copy, from_variables, what)
            assert_bits_equal(strided(False, True), from_variables, what)
            assert_bits_equal(_run(hip, device, x, dev, copy.blob, ob, n_out, k_in, act), from_variables, what)


def test_layer_reads_a_column_slice_where_it_lies(hip, device, oracle):
    """LinearGQ(dim=0).build on a decode batch that is a column slice of a wider matrix: no gather, the result of the
    gathered call bit for bit; a slice of more than 16 rows is gathered as before."""
    from popxl_addons.layers.linear_gq import LinearGQ

    n_out, k_in = 4096, 4096
    layer = LinearGQ(n_out, bias=False, group_size=64, dim=0)
    layer.init_variables(k_in, torch.float16, device)
    (p, s, b), _, w_dec = _weight(hip, device, oracle, n_out, k_in, 31)
    v = layer.variables
    v.weight_compressed.data.copy_(p.reshape(v.weight_compressed.shape))
    v.weight_decompression_scale.data.copy_(s.reshape(v.weight_decompression_scale.shape))
    v.weight_decompression_bias.data.copy_(b.reshape(v.weight_decompression_bias.shape))
    for with_copy in (False, True):
        if with_copy:
            layer.prepack_for_decode()
        for m_rows in (4, 40):
            wide = to_dev(activations(m_rows, k_in + 512, 80 + m_rows), device)
            part = wide[:, 256 : 256 + k_in]
            assert not part.is_contiguous()
            y = layer(part).cpu().numpy()
            assert_bits_equal(y, layer(part.contiguous()).cpu().numpy(), (with_copy, m_rows))
            assert_close(y, oracle.np_linear(part.cpu().numpy(), w_dec, None), (with_copy, m_rows))
    layer._decode_copy = None


def test_without_the_copy_it_is_the_workspace_entry_point(hip, device, oracle):
    n_out, k_in, m_rows = 4096, 4096, 256
    dev, _, _ = _weight(hip, device, oracle, n_out, k_in, 31)
    x = activations(m_rows, k_in, 34)
    xd = to_dev(x, device)
    y = torch.empty((m_rows, n_out), dtype=torch.float16, device=device)
    hip.call("gq_linear_act_ws_f16", xd.data_ptr(), m_rows, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(), 0,
             y.data_ptr(), n_out, k_in, 64, 1, 0, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert_bits_equal(_run(hip, device, x, dev, None, None, n_out, k_in, 1), y.cpu().numpy(), "blob == NULL")


def test_rejected_arguments(hip, device, oracle):
    dev, copy, _ = _weight(hip, device, oracle, 72, 512, 31)
    x = activations(40, 512, 35)
    with pytest.raises(GQHipError) as e:  # a copy that is not 16-byte aligned
        _run(hip, device, x, dev, copy.blob[8:], None, 72, 512, 0)
    assert e.value.code == GQ_ERR_MISALIGNED
    # no streaming layout exists for group size 32 or for 320 input features: a copy cannot be meant
    packed, scale, bias = group_quantize_compress_numpy(normal_weight(64, 320, 3), 64)
    odd = tuple(to_dev(a, device) for a in (packed, scale, bias))
    with pytest.raises(GQHipError) as e:
        _run(hip, device, activations(40, 320, 36), odd, copy.blob, None, 64, 320, 0)
    assert e.value.code == GQ_ERR_UNSUPPORTED and "streaming layout" in str(e.value)
    # the copy alone takes a 16-byte aligned x; some of the variables without the others are an error
    xd = to_dev(activations(41, 512, 37), device)
    y = torch.empty((40, 72), dtype=torch.float16, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(GQHipError) as e:
        hip.call("gq_linear_p_act_f16", xd.data_ptr() + 2, 40, 0, 0, 0, copy.blob.data_ptr(), 0, y.data_ptr(), 72, 512, 64, 0, 0, 0, stream)
    assert e.value.code == GQ_ERR_MISALIGNED and "16-byte" in str(e.value)
    with pytest.raises(GQHipError) as e:
        hip.call("gq_linear_p_act_f16", xd.data_ptr(), 40, 0, dev[1].data_ptr(), dev[2].data_ptr(), copy.blob.data_ptr(), 0, y.data_ptr(),
                 72, 512, 64, 0, 0, 0, stream)
    assert e.value.code == GQ_ERR_NULL_POINTER


def test_layer_with_the_copy(hip, device, oracle):
    """LinearGQ(dim=0) after prepack_for_decode(): prefill batches read the copy, decode batches the
    variables; the same results as before the copy was made."""
    from popxl_addons.layers.linear_gq import LinearGQ

    n_out, k_in = 4096, 4096
    layer = LinearGQ(n_out, bias=True, group_size=64, dim=0)
    layer.init_variables(k_in, torch.float16, device)
    (p, s, b), _, w_dec = _weight(hip, device, oracle, n_out, k_in, 31)
    ob = np.random.default_rng(37).normal(0, 1, (n_out,)).astype(np.float16)
    v = layer.variables
    v.weight_compressed.data.copy_(p.reshape(v.weight_compressed.shape))
    v.weight_decompression_scale.data.copy_(s.reshape(v.weight_decompression_scale.shape))
    v.weight_decompression_bias.data.copy_(b.reshape(v.weight_decompression_bias.shape))
    v.bias.data.copy_(to_dev(ob, device))
    for m_rows in (4, 300):
        x = activations(m_rows, k_in, 38 + m_rows)
        before = layer(to_dev(x, device)).cpu().numpy()
        copy = layer.prepack_for_decode()
        assert copy.layout == "nk" and layer._decode_copy is copy
        after = layer(to_dev(x, device)).cpu().numpy()
        assert_bits_equal(after, before, m_rows)
        assert_close(after, oracle.np_linear(x, w_dec, ob), m_rows)
        layer._decode_copy = None
