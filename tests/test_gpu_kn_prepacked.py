"""GPU parity of the decode path of LinearGQ's default layout (groups along the OUTPUT features,
popxl_addons/layers/linear_gq.py:26, 59-62, 99-109) on the kn streaming layout: gq_gemv_kn_prepack_f16
makes the derived copy, gq_linear_knp_act_f16 and sequence entries marked GQ_DESC_KN_LAYOUT read it.
Oracle: float32/float64 matmul over the oracle-decompressed weight; contract max|y - y_ref| / max|y_ref|
<= 1e-2, regression bound 2e-3 for the whole result and for every output column."""
import numpy as np
import pytest
import torch

from gq_testlib import activations, assert_bits_equal, to_dev
from popxl_addons.layers.linear_gq import LinearGQ
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy
from test_gpu_fused import assert_close

pytestmark = pytest.mark.gpu

_WEIGHTS = {}


def _weight(oracle, device, k_in, n_out, seed, spread=False):
    """(blob, variables on the device, oracle-decompressed weight transposed to [n_out, k_in])."""
    from popxl_addons._gq_hip import prepack_gemv_kn

    key = (k_in, n_out, seed, spread)
    if key not in _WEIGHTS:
        rng = np.random.default_rng(seed)
        w = rng.normal(0, 0.02, (k_in, n_out)).astype(np.float32)
        if spread:  # scales and biases that differ a lot from group to group and from row to row
            w *= np.exp(rng.normal(0, 1.5, (k_in, 1))).astype(np.float32)
            w += rng.normal(0, 0.05, (k_in, n_out // 64)).astype(np.float32).repeat(64, axis=1)
        packed, scale, bias = group_quantize_compress_numpy(w.astype(np.float16), 64)
        w_dec_t = np.ascontiguousarray(oracle.np_decompress(packed, scale, bias).T)
        _WEIGHTS[key] = (packed, scale, bias, w_dec_t)
    packed, scale, bias, w_dec_t = _WEIGHTS[key]
    variables = tuple(to_dev(a, device) for a in (packed, scale, bias))
    return prepack_gemv_kn(*variables), variables, w_dec_t


def test_prepack_layout_word_for_word(hip, device):
    """The blob against a numpy restatement of the layout: unit (g, c) = 64 outputs x 512 input features;
    16 KiB of codes as [row block j][load s][lane (kc, r)][word w], code e of a word in nibble
    (3,7,2,6,1,5,0,4)[e], then the 512 scales and the 512 biases of the group."""
    from popxl_addons._gq_hip import prepack_gemv_kn

    k_in, n_out = 1024, 192
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 16, (k_in, n_out)).astype(np.uint32)
    c4 = codes.reshape(k_in, n_out // 64, 16, 4)
    packed = ((c4[..., 0] << 12) | (c4[..., 1] << 8) | (c4[..., 2] << 4) | c4[..., 3]).astype(np.uint16)
    scale = rng.normal(0, 1, (k_in, n_out // 64, 1)).astype(np.float16)
    bias = rng.normal(0, 1, (k_in, n_out // 64, 1)).astype(np.float16)
    blob = prepack_gemv_kn(*(to_dev(a, device) for a in (packed, scale, bias)))
    assert blob.layout == "kn" and (blob.n_out, blob.k_in, blob.group_size) == (n_out, k_in, 64)
    raw = blob.blob.cpu().numpy()
    assert raw.size == (n_out // 64) * (k_in // 512) * 18432
    units = raw.reshape(n_out // 64, k_in // 512, 18432)
    nibble = np.array([3, 7, 2, 6, 1, 5, 0, 4])
    for g in range(n_out // 64):
        for c in range(k_in // 512):
            words = units[g, c, :16384].view(np.uint32).reshape(4, 4, 4, 16, 4)  # [j][s][kc][r][w]
            # codes[k][n] for k = 512 c + 128 s + 32 kc + 8 w + e, n = 64 g + 16 j + r
            block = codes[512 * c : 512 * (c + 1), 64 * g : 64 * (g + 1)].reshape(4, 4, 4, 8, 4, 16)  # [s][kc][w][e][j][r]
            want = (block << (4 * nibble)[None, None, None, :, None, None]).sum(axis=3).transpose(3, 0, 1, 4, 2)  # [j][s][kc][r][w]
            assert np.array_equal(words, want.astype(np.uint32)), (g, c)
            assert np.array_equal(units[g, c, 16384:17408].view(np.uint16), scale[512 * c : 512 * (c + 1), g, 0].view(np.uint16))
            assert np.array_equal(units[g, c, 17408:].view(np.uint16), bias[512 * c : 512 * (c + 1), g, 0].view(np.uint16))


@pytest.mark.parametrize("k_in,n_out", [(4096, 4096), (4096, 16384), (16384, 4096), (4096, 12288), (512, 64), (1536, 320), (5120, 4160)])
@pytest.mark.parametrize("m_rows", [1, 2, 3, 4, 5, 8, 13, 16])
def test_decode_shapes(hip, device, oracle, k_in, n_out, m_rows):
    """The layer shapes of the 6B stack (benchmark configurations 3 and 5 in the default layout), the
    fused q|k|v width, and small and ragged shapes: fewer chunks than waves, group counts that fill
    no whole round of workgroups."""
    from popxl_addons._gq_hip import linear_knp

    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 11)
    rng = np.random.default_rng(100 + m_rows)
    x = activations(m_rows, k_in, 12 + m_rows)
    for with_bias in (False, True):
        ob = rng.normal(0, 1, (n_out,)).astype(np.float16) if with_bias else None
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        linear_knp(to_dev(x, device), blob, None if ob is None else to_dev(ob, device), None, y)
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, ob), (k_in, n_out, m_rows, with_bias))


@pytest.mark.parametrize("k_in,n_out", [(4096, 4096), (4096, 16384), (16384, 4096), (512, 64), (1536, 320), (1024, 4160)])
@pytest.mark.parametrize("m_rows", [17, 31, 33, 64, 128, 200, 512])
def test_prefill_shapes(hip, device, oracle, k_in, n_out, m_rows):
    """More than 16 rows from the same copy: two passes of the decode kernel up to 32 rows, then the
    pipelined MFMA kernel with every tile shape it has (64 x 64 ... 256 x 256, by batch and width),
    ragged batches and widths that fill no whole tile."""
    from popxl_addons._gq_hip import linear_knp

    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 11)
    x = activations(m_rows, k_in, 14 + m_rows)
    ob = np.random.default_rng(200 + m_rows).normal(0, 1, (n_out,)).astype(np.float16)
    y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    linear_knp(to_dev(x, device), blob, to_dev(ob, device), None, y)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, ob), (k_in, n_out, m_rows))


def test_benchmark_prefill_batches(hip, device, oracle):
    """Benchmark configuration 4 in the default layout: 4096 -> 16384 at 1024 and 2048 rows (the 256 x 128 and
    256 x 256 tiles), with an activation epilogue."""
    from popxl_addons._gq_hip import linear_knp

    k_in, n_out = 4096, 16384
    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 11)
    for m_rows in (1024, 2048):
        x = activations(m_rows, k_in, 15)
        y = linear_knp(to_dev(x, device), blob, None, "relu")
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, None, "relu"), m_rows)


@pytest.mark.parametrize("m_rows", [64, 300])
def test_prefill_uneven_scales_and_biases(hip, device, oracle, m_rows):
    """Scales and biases that vary by orders of magnitude between input features, through the MFMA
    pipeline (every input feature applies its own to the codes)."""
    from popxl_addons._gq_hip import linear_knp

    k_in, n_out = 4096, 1024
    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 21, spread=True)
    x = activations(m_rows, k_in, 23)
    y = linear_knp(to_dev(x, device), blob)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, None), m_rows)


@pytest.mark.parametrize("m_rows", [1, 8])
def test_uneven_scales_and_biases(hip, device, oracle, m_rows):
    """Scales and biases that vary by orders of magnitude between input features: the activations are
    multiplied by the scales before the matrix instruction, in binary16 -- the result must stay within
    the regression bound of every output column."""
    from popxl_addons._gq_hip import linear_knp

    k_in, n_out = 4096, 1024
    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 21, spread=True)
    x = activations(m_rows, k_in, 22)
    y = linear_knp(to_dev(x, device), blob)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, None), m_rows)


@pytest.mark.parametrize("activation", ["relu", "gelu_tanh"])
def test_activation_epilogue(hip, device, oracle, activation):
    from popxl_addons._gq_hip import linear_knp

    k_in, n_out, m_rows = 1024, 2048, 4
    blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 31)
    x = activations(m_rows, k_in, 32)
    ob = np.random.default_rng(33).normal(0, 1, (n_out,)).astype(np.float16)
    y = linear_knp(to_dev(x, device), blob, to_dev(ob, device), activation)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.np_linear(x, w_dec_t, ob, activation), activation)


def test_agrees_with_the_kernel_on_the_variables(hip, device, oracle):
    """The same problem through gq_linear_kn_act_f16 (the three variables) and through the blob."""
    from popxl_addons._gq_hip import linear_knp

    k_in, n_out, m_rows = 4096, 4096, 4
    blob, (packed, scale, bias), w_dec_t = _weight(oracle, device, k_in, n_out, 11)
    x = to_dev(activations(m_rows, k_in, 41), device)
    need = hip.load().gq_linear_kn_workspace_bytes(m_rows, n_out, k_in, 64)
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=device)
    y_vars = torch.empty((m_rows, n_out), dtype=torch.float16, device=device)
    hip.call("gq_linear_kn_act_f16", x.data_ptr(), m_rows, packed.data_ptr(), scale.data_ptr(), bias.data_ptr(), 0, y_vars.data_ptr(),
             n_out, k_in, 64, 0, ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    y_blob = linear_knp(x, blob)
    torch.cuda.synchronize()
    ref = oracle.np_linear(x.cpu().numpy(), w_dec_t, None)
    assert_close(y_vars.cpu().numpy(), ref, "variables")
    assert_close(y_blob.cpu().numpy(), ref, "blob")


@pytest.mark.parametrize("k_in,n_out", [(4096, 4096), (4096, 16384), (16384, 4096), (1536, 320)])
@pytest.mark.parametrize("m_rows", [1, 4, 8, 16])
def test_rows_of_x_a_stride_apart(hip, device, oracle, k_in, n_out, m_rows):
    """gq_linear_knp_strided_f16: x as a column slice of a wider matrix gives the bits of the call on the gathered
    x (the same kernel reads it where it lies), and the oracle's result."""
    from popxl_addons._gq_hip import linear_knp

    copy, _, w_dec_t = _weight(oracle, device, k_in, n_out, 11)
    ob = np.random.default_rng(91).normal(0, 1, (n_out,)).astype(np.float16)
    wide = to_dev(activations(m_rows, k_in + 264, 90 + m_rows), device)
    for offset in (0, 136):
        part = wide[:, offset : offset + k_in]
        assert not part.is_contiguous() or m_rows == 1
        y = linear_knp(part, copy, to_dev(ob, device), "relu").cpu().numpy()
        gathered = linear_knp(part.contiguous(), copy, to_dev(ob, device), "relu").cpu().numpy()
        assert_bits_equal(y, gathered, (k_in, n_out, m_rows, offset))
        assert_close(y, oracle.np_linear(part.cpu().numpy(), w_dec_t, ob, "relu"), (k_in, n_out, m_rows, offset))


def test_rejected_arguments(hip, device):
    from popxl_addons._gq_hip import GQ_ERR_MISALIGNED, GQ_ERR_UNSUPPORTED, GQHipError

    lib = hip.load()
    assert lib.gq_gemv_kn_prepacked_bytes(4096, 4096, 64) == 4096 * 4096 * 9 // 16
    assert lib.gq_gemv_kn_prepacked_bytes(0, 4096, 64) == 0
    for n_out, k_in, gs in ((4096, 4096, 32), (4096, 4000, 64), (4100, 4096, 64)):
        assert lib.gq_gemv_kn_prepacked_bytes(n_out, k_in, gs) == GQ_ERR_UNSUPPORTED
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(GQHipError) as e:  # a group size the layout does not have
        hip.call("gq_linear_knp_act_f16", buf.data_ptr(), 17, buf.data_ptr(), 0, buf.data_ptr(), 64, 512, 32, 0, stream)
    assert e.value.code == GQ_ERR_UNSUPPORTED
    with pytest.raises(GQHipError) as e:
        hip.call("gq_linear_knp_act_f16", buf.data_ptr() + 2, 1, buf.data_ptr(), 0, buf.data_ptr(), 64, 512, 64, 0, stream)
    assert e.value.code == GQ_ERR_MISALIGNED
    hip.call("gq_linear_knp_act_f16", 0, 0, 0, 0, 0, 64, 512, 64, 0, stream)  # an empty batch: nothing to do


@pytest.mark.parametrize("dim", [-1, 1])
def test_layer_serves_decode_batches_from_the_copy(hip, device, oracle, dim):
    """LinearGQ with the reference's default dim: after prepack_for_decode() batches of up to 16 rows
    read the derived copy, larger ones the variables; load_weights renews the copy."""
    torch.manual_seed(4)
    layer = LinearGQ(1024, bias=True, group_size=64, dim=dim)
    variables = layer.init_variables(1024, torch.float16, device)
    refs = []
    for round_ in range(2):
        nn_layer = torch.nn.Linear(1024, 1024, bias=True)
        layer.load_weights(LinearGQ.torch_mapping(variables, nn_layer, dtype=torch.float16, group_size=64, dim=dim))
        if round_ == 0:
            copy = layer.prepack_for_decode()
            assert copy.layout == "kn" and layer._decode_copy is copy
        else:
            assert layer._decode_copy is not None and layer._decode_copy is not copy  # renewed by load_weights
        v = layer.variables
        w_dec_t = np.ascontiguousarray(oracle.np_decompress(v.weight_compressed.data.cpu().numpy(),
                                                            v.weight_decompression_scale.data.cpu().numpy(),
                                                            v.weight_decompression_bias.data.cpu().numpy()).T)
        for batch in ((1,), (2, 3), (16,), (40,)):
            x = np.random.default_rng(50 + len(refs)).normal(0, 1, (*batch, 1024)).astype(np.float16)
            y = layer(to_dev(x, device), activation="relu").cpu().numpy()
            ref = oracle.np_linear(x.reshape(-1, 1024), w_dec_t, v.bias.data.cpu().numpy(), "relu").reshape(*batch, 1024)
            assert_close(y, ref, (round_, batch))
            refs.append(ref)
        # a decode batch that is a column slice of a wider matrix is read where it lies: the gathered call's bits
        wide = to_dev(np.random.default_rng(60 + round_).normal(0, 1, (5, 1024 + 512)).astype(np.float16), device)
        part = wide[:, 256 : 256 + 1024]
        assert_bits_equal(layer(part).cpu().numpy(), layer(part.contiguous()).cpu().numpy(), (round_, "slice"))


@pytest.mark.parametrize("m_rows", [1, 8])
def test_sequence_entries_in_the_default_layout(hip, device, oracle, m_rows):
    """A chain of GEMVs whose weights are in the kn streaming layout (what a stack of default-constructed
    LinearGQ layers gives), mixed with an entry in the other layout: every entry against the oracle on
    the inputs the device had, twice."""
    from popxl_addons._gq_hip import GemvSequence
    from test_gpu_fused import _full_size_weight

    shapes = [(4096, 4096), (16384, 4096), (4096, 16384)]  # (n_out, k_in)
    seq = GemvSequence(device)
    x0 = activations(m_rows, 4096, 61)
    x_in, plan, outs = to_dev(x0, device), [], []
    for i, (n_out, k_in) in enumerate(shapes):
        blob, _, w_dec_t = _weight(oracle, device, k_in, n_out, 60 + i)
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        seq.add(x_in, blob, None, None, y, None, wait_previous=i > 0, activation="relu" if i == 1 else None)
        plan.append((x_in, w_dec_t, y, "relu" if i == 1 else None))
        x_in = y
    packed, scale, bias, w_dec = _full_size_weight(oracle, 4096, 4096, 64)  # groups along the input features
    y = torch.full((m_rows, 4096), float("nan"), dtype=torch.float16, device=device)
    seq.add(x_in, to_dev(packed, device), to_dev(scale, device), to_dev(bias, device), y, None, wait_previous=True)
    plan.append((x_in, w_dec, y, None))
    for run in range(2):
        for _, _, y, _ in plan:
            y.fill_(float("nan"))
        seq.run()
        seq.check()
        for i, (x_dev, w, y, act) in enumerate(plan):
            assert_close(y.cpu().numpy(), oracle.np_linear(x_dev.cpu().numpy(), w, None, act), (run, i))
