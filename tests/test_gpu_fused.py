"""GPU parity of the fused dequant-GEMV / GEMM entry points (C ABI: gq_gemv_f16, gq_gemm_f16,
gq_linear_f16) against a float32 matmul over the oracle-decompressed weight.
Tolerance: max|y_gpu - y_ref| / max|y_ref| <= 1e-2."""
import numpy as np
import pytest
import torch

from gq_testlib import activations, normal_weight, normalised_error, to_dev
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy

pytestmark = pytest.mark.gpu
TOL = 1e-2  # the contract: max|y_gpu - y_ref| / max|y_ref|
# Regression bound, well above what the kernels deliver (about 6e-4: the weight is rounded to fp16
# once instead of twice, the sums are fp32) and well below the contract: the whole result AND every
# output column (one weight row, i.e. one group of scales, however small its values) must be within
# 2e-3 of the largest reference value.
REGRESSION_TOL = 2e-3


def assert_close(y_gpu, y_ref, what=""):
    y_gpu = np.asarray(y_gpu, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    assert y_gpu.shape == y_ref.shape, (what, y_gpu.shape, y_ref.shape)
    assert np.isfinite(y_gpu).all(), what
    top = max(np.abs(y_ref).max(), 1e-30)
    err = np.abs(y_gpu - y_ref)
    assert err.max() / top <= TOL, (what, err.max() / top)
    worst_column = err.reshape(-1, y_ref.shape[-1]).max(axis=0)
    bad = np.flatnonzero(worst_column > REGRESSION_TOL * top)
    assert bad.size == 0, (what, "columns", bad[:8], (worst_column[bad[:8]] / top))


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


_CASE_WEIGHTS = {}


def _case(oracle, n_out, k_in, gs, m_rows, seed, with_bias):
    key = (n_out, k_in, gs, seed)  # (large weights take seconds to compress and decompress on the host: once per session)
    if key not in _CASE_WEIGHTS:
        packed, scale, bias = group_quantize_compress_numpy(normal_weight(n_out, k_in, seed), gs)
        _CASE_WEIGHTS[key] = (packed, scale, bias, oracle.np_decompress(packed, scale, bias))
    packed, scale, bias, w_dec = _CASE_WEIGHTS[key]
    x = activations(m_rows, k_in, seed + 1)
    out_bias = np.random.default_rng(seed + 2).normal(0, 1, (n_out,)).astype(np.float16) if with_bias else None
    y_ref = oracle.np_linear(x, w_dec, out_bias)
    return x, packed, scale, bias, out_bias, y_ref


@pytest.mark.parametrize("n_out,k_in", [(4096, 4096), (16384, 4096), (4096, 16384), (20480, 4096), (12288, 4096)])
@pytest.mark.parametrize("m_rows", [1, 2, 3, 4, 8, 16])
def test_gemv_benchmark_shapes(hip, device, oracle, n_out, k_in, m_rows):
    """Benchmark configurations 3 and 5: decode batches on the layer shapes of the 6B stack, on a weight
    large enough for the single call to go through the persistent kernel at up to four rows
    (20480 x 4096) and on one whose row blocks do not divide evenly over the compute units (12288 x 4096)."""
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 7, with_bias)
        y = _call(hip, "gq_gemv_f16", x, packed, scale, bias, ob, n_out, k_in, 64, device)
        assert_close(y, y_ref, (n_out, k_in, m_rows, with_bias))


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
        # group 64, k_in % 512 == 0: x goes through LDS (1, 4, 8 or 16 rows), with 1, 2 or 4 row blocks per wave
        (40, 512, 64, 1),
        (8200, 1024, 64, 1),
        (8200, 512, 64, 7),
        (8200, 1536, 64, 13),
        (16400, 512, 64, 3),
        (16400, 1024, 64, 8),
        (16400, 512, 64, 16),
        (100, 8192, 64, 2),  # several chunks per wave
        (100, 8192, 64, 11),
        (300, 11008, 64, 5),  # a last chunk of 256 features (21 whole chunks before it)
        (64, 896, 64, 16),
        (8200, 640, 64, 1),
        # the same with groups of 128 (8-byte scale / bias loads) and of 32 and 256 (2-byte loads)
        (48, 1024, 128, 5),
        (8200, 512, 128, 2),
        (33, 512, 32, 9),
        (16400, 1024, 256, 1),
    ],
)
def test_gemv_edge_shapes(hip, device, oracle, n_out, k_in, gs, m_rows):
    for with_bias in (False, True):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 11, with_bias)
        for entry in ("gq_gemv_f16", "gq_linear_f16"):
            y = _call(hip, entry, x, packed, scale, bias, ob, n_out, k_in, gs, device)
            assert_close(y, y_ref, (entry, with_bias))


def _call_offset(hip, entry, x, packed, scale, bias, out_bias, n_out, k_in, gs, device, offsets):
    """The same call with operands placed `offsets[name]` bytes past a 256-byte aligned address."""
    def place(a, off):
        raw = np.ascontiguousarray(a).view(np.uint8).reshape(-1)
        buf = torch.zeros(raw.size + 256, dtype=torch.uint8, device=device)
        buf[off : off + raw.size] = torch.from_numpy(raw).to(device)
        return buf, buf.data_ptr() + off

    keep, ptr = {}, {}
    for name, a in (("x", x), ("packed", packed), ("scale", scale), ("bias", bias)):
        keep[name], ptr[name] = place(a, offsets.get(name, 0))
    od = None if out_bias is None else to_dev(out_bias, device)
    y = torch.full((x.shape[0], n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call(entry, ptr["x"], x.shape[0], ptr["packed"], ptr["scale"], ptr["bias"], 0 if od is None else od.data_ptr(),
             y.data_ptr(), n_out, k_in, gs, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("gs", [64, 128])
@pytest.mark.parametrize("m_rows", [1, 8])
def test_gemv_alignment_fallbacks(hip, device, oracle, gs, m_rows):
    """The fast GEMV kernels read scale / bias with 16-byte (group 64) or 8-byte (group 128) loads and
    x / packed with 16-byte loads: operands that are only 2-, 4- or 8-byte aligned take the
    kernels with narrower loads and give the same result."""
    n_out, k_in = 520, 1024
    x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 3, True)
    y_fast = _call(hip, "gq_gemv_f16", x, packed, scale, bias, ob, n_out, k_in, gs, device)
    assert_close(y_fast, y_ref, "aligned")
    for offsets in ({"scale": 2}, {"bias": 2}, {"scale": 4, "bias": 8}, {"scale": 8}, {"x": 2}, {"packed": 2},
                    {"x": 8, "packed": 4, "scale": 2, "bias": 6}):
        y = _call_offset(hip, "gq_gemv_f16", x, packed, scale, bias, ob, n_out, k_in, gs, device, offsets)
        assert_close(y, y_ref, offsets)
        assert normalised_error(y, y_fast.astype(np.float32)) <= REGRESSION_TOL, offsets


@pytest.mark.parametrize("m_rows", [1, 2, 5])
def test_gemv_outlier_activations_and_uneven_groups(hip, device, oracle, m_rows):
    """Activations with a few values hundreds of times the rest, and weight rows whose groups differ in spread by
    a factor of 250 and sit off zero (large biases): the kernels that apply scale and bias to group sums take the
    codes' offsets (64 and 1024 per weight) out of sums that such activations dominate.  One and two rows run
    that arithmetic, five rows the kernel that expands every weight; from the variables and from the copy."""
    from popxl_addons._gq_hip import prepack_gemv

    n_out, k_in = 1000, 4096
    rng = np.random.default_rng(77)
    spread = np.exp(rng.uniform(np.log(2e-4), np.log(5e-2), (n_out, k_in // 64, 1)))
    centre = rng.normal(0, 0.05, (n_out, k_in // 64, 1))
    w = (rng.normal(0, 1, (n_out, k_in // 64, 64)) * spread + centre).reshape(n_out, k_in).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, 64)
    w_dec = oracle.np_decompress(packed, scale, bias)
    x = activations(m_rows, k_in, 78)
    where = rng.choice(k_in, 12, replace=False)
    x[:, where] = (rng.choice([-1.0, 1.0], (m_rows, 12)) * rng.uniform(100, 600, (m_rows, 12))).astype(np.float16)
    y_ref = oracle.np_linear(x, w_dec, None)
    assert_close(_call(hip, "gq_gemv_f16", x, packed, scale, bias, None, n_out, k_in, 64, device), y_ref, "variables")
    dev = tuple(to_dev(a, device) for a in (packed, scale, bias))
    copy = prepack_gemv(*dev)
    y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call("gq_linear_p_act_f16", to_dev(x, device).data_ptr(), m_rows, 0, 0, 0, copy.blob.data_ptr(), 0, y.data_ptr(), n_out, k_in, 64,
             0, 0, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), y_ref, "copy")


@pytest.mark.parametrize("m_rows", [128, 512, 2048])
def test_gemm_benchmark_shapes(hip, device, oracle, m_rows):
    """Benchmark configuration 4: prefill batches on the [16384 x 4096] weight."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, 16384, 4096, 64, m_rows, 21, m_rows == 512)
    y = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, 16384, 4096, 64, device)
    assert_close(y, y_ref, m_rows)


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
            assert_close(y, y_ref, (entry, with_bias))


@pytest.mark.parametrize("n_out,k_in,m_rows", [(4096, 4096, 17), (4096, 4096, 40), (4096, 4096, 64), (4096, 4096, 96),
                                               (4096, 16384, 90), (16384, 4096, 32), (16384, 4096, 48), (4104, 4096, 33)])
def test_linear_mid_batches(hip, device, oracle, n_out, k_in, m_rows):
    """gq_linear_f16 between the GEMV's 16 rows and full GEMM tiles: on large weights it runs passes of
    the GEMV kernel over 16 rows each where those are expected to beat the mostly empty GEMM tiles
    (some of these cases), the GEMM kernel otherwise; either way the result is that of gq_gemm_f16."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 17, True)
    y = _call(hip, "gq_linear_f16", x, packed, scale, bias, ob, n_out, k_in, 64, device)
    assert_close(y, y_ref, (n_out, k_in, m_rows))
    y_gemm = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, n_out, k_in, 64, device)
    assert normalised_error(y, y_gemm.astype(np.float32)) <= REGRESSION_TOL


@pytest.mark.parametrize("n_out,k_in,m_rows", [(4104, 384, 1030), (4104, 384, 2060), (4104, 512, 300), (8200, 256, 777)])
def test_gemm_large_tiles_on_ragged_problems(hip, device, oracle, n_out, k_in, m_rows):
    """The tile shape is chosen by expected time (tiles per compute unit x time per tile): these ragged
    problems are large enough for the 256 x 128 tiles (1030 rows), the 256 x 256 tiles (2060 and 777
    rows) and 128 x 64 tiles with K split between two groups of waves (300 rows)."""
    x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, 64, m_rows, 47, True)
    y = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, n_out, k_in, 64, device)
    assert_close(y, y_ref, (n_out, k_in, m_rows))


def test_linear_with_workspace(hip, device, oracle):
    """gq_linear_act_ws_f16: on weights with few outputs the workgroups of an output tile divide the
    input features between them and add their accumulators through the workspace.  One workspace
    serves problems of several shapes one after the other (its arrival counters are back at zero after
    every call); ragged tiles, every tile shape that the choice reaches here, an activation; the
    result is the oracle's, and that of the call without a workspace to a few roundings."""
    lib = hip.load()
    cases = [(4096, 16384, 128), (4096, 16384, 300), (4096, 4096, 64), (4096, 4096, 256), (4104, 2048, 100), (2056, 8192, 520),
             (1000, 4096, 40)]
    needs = [lib.gq_gemm_workspace_bytes(m, n, k, 64) for n, k, m in cases]
    assert sum(need > 16384 for need in needs) >= 5, needs  # (a problem for which dividing K does not pay asks for none)
    assert lib.gq_gemm_workspace_bytes(16, 4096, 16384, 64) == 0 and lib.gq_gemm_workspace_bytes(2048, 16384, 4096, 64) == 0
    ws = torch.zeros(max(needs), dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    for (n_out, k_in, m_rows), need in zip(cases, needs):
        x, packed, scale, bias, ob, _ = _case(oracle, n_out, k_in, 64, m_rows, 29, True)
        w_dec = _CASE_WEIGHTS[(n_out, k_in, 64, 29)][3]
        y_ref = oracle.np_linear(x, w_dec, ob, "gelu_tanh")
        xd, pd, sd, bd, od = (to_dev(a, device) for a in (x, packed, scale, bias, ob))
        got = []
        for workspace in (ws, None):
            y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
            hip.call("gq_linear_act_ws_f16", xd.data_ptr(), m_rows, pd.data_ptr(), sd.data_ptr(), bd.data_ptr(), od.data_ptr(),
                     y.data_ptr(), n_out, k_in, 64, 2, 0 if workspace is None else workspace.data_ptr(),
                     0 if workspace is None else workspace.numel(), stream)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), y_ref, (n_out, k_in, m_rows, workspace is not None))
            got.append(y.cpu().numpy())
        assert not ws[:16384].any(), "arrival counters must be back at zero"
        assert normalised_error(got[0], got[1].astype(np.float32)) <= REGRESSION_TOL


@pytest.mark.parametrize("m_rows", [33, 70, 100, 260, 300, 1030])
def test_gemm_every_kernel_shape(hip, device, oracle, m_rows):
    """Small ragged problems on the pipelined kernel's 128 x 64 tiles (with K split between two groups
    of waves where k_in is a multiple of 256), the LDS-staged tile kernel (odd number of groups per
    row, or scale / bias that are only 2-byte aligned) and the generic kernel (group 16)."""
    for n_out, k_in, gs in ((300, 1024, 64), (130, 448, 32), (96, 192, 64), (200, 768, 128), (72, 320, 64), (40, 96, 16)):
        x, packed, scale, bias, ob, y_ref = _case(oracle, n_out, k_in, gs, m_rows, 41, True)
        y = _call(hip, "gq_gemm_f16", x, packed, scale, bias, ob, n_out, k_in, gs, device)
        assert_close(y, y_ref, (n_out, k_in, gs, m_rows))
    x, packed, scale, bias, ob, y_ref = _case(oracle, 300, 1024, 64, m_rows, 43, False)
    y = _call_offset(hip, "gq_gemm_f16", x, packed, scale, bias, ob, 300, 1024, 64, device, {"scale": 2, "bias": 2})
    assert_close(y, y_ref, "tile kernel")


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


_FULL_SIZE_WEIGHTS = {}


def _full_size_weight(oracle, n_out, k_in, seed):
    """(packed, scale, bias, decompressed) of a seeded N(0, 1 / k_in) weight -- a scale that keeps a
    chain of layers at unit magnitude; made once per session (a full-size weight takes seconds to draw,
    compress and decompress on the host, and several tests and their cases use the same ones)."""
    key = (n_out, k_in, seed)
    if key not in _FULL_SIZE_WEIGHTS:
        w = np.random.default_rng(seed).normal(0, 1.0 / np.sqrt(k_in), (n_out, k_in)).astype(np.float16)
        packed, scale, bias = group_quantize_compress_numpy(w, 64)
        _FULL_SIZE_WEIGHTS[key] = (packed, scale, bias, oracle.np_decompress(packed, scale, bias))
    return _FULL_SIZE_WEIGHTS[key]


def _sequence_case(hip, device, oracle, shapes, m_rows, chained, seed=50):
    """Entries of the given (n_out, k_in) shapes; `chained`: entry i reads entry i-1's output."""
    from popxl_addons._gq_hip import GemvSequence

    rng = np.random.default_rng(seed)
    seq = GemvSequence(device)
    refs, outs = [], []
    x_host = activations(m_rows, shapes[0][1], seed)
    x_dev = to_dev(x_host, device)
    for i, (n_out, k_in) in enumerate(shapes):
        packed, scale, bias, w_dec = _full_size_weight(oracle, n_out, k_in, 1000 * seed + i)
        ob = rng.normal(0, 0.1, (n_out,)).astype(np.float16) if i % 2 else None
        if chained and i > 0:
            assert k_in == shapes[i - 1][0]
            x_host = refs[-1].astype(np.float16)  # what the device chain holds up to fp16 rounding
            x_in = outs[-1]
        else:
            x_host = activations(m_rows, k_in, seed + i)
            x_in = to_dev(x_host, device)
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        seq.add(x_in, to_dev(packed, device), to_dev(scale, device), to_dev(bias, device), y,
                None if ob is None else to_dev(ob, device), wait_previous=chained and i > 0)
        refs.append(oracle.np_linear(x_host, w_dec, ob))
        outs.append(y)
    return seq, refs, outs


@pytest.mark.parametrize("m_rows", [1, 4, 8])
def test_gemv_sequence_independent_entries(hip, device, oracle, m_rows):
    """Every entry of a sequence equals the single-call result (benchmark configuration 5 shapes,
    ragged row counts, a k_in that is not a multiple of 4096)."""
    shapes = [(4096, 4096), (4096, 4096), (1000, 4096), (16384, 4096), (4096, 16384), (16, 512), (5000, 1536), (40, 8192)]
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, m_rows, chained=False)
    for _ in range(2):  # twice: the progress counters must be back at zero after a run
        for y in outs:
            y.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        for (n_out, k_in), y, ref in zip(shapes, outs, refs):
            yy = y.cpu().numpy()
            assert np.isfinite(yy).all(), (n_out, k_in)
            assert_close(yy, ref, (n_out, k_in))


@pytest.mark.parametrize("m_rows", [1, 4])
def test_gemv_sequence_chained_entries(hip, device, oracle, m_rows):
    """wait_previous: each entry consumes the previous entry's output (other compute units wrote it)."""
    shapes = [(4096, 4096), (2048, 4096), (4096, 2048), (16384, 4096), (4096, 16384), (512, 4096)]
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, m_rows, chained=True)
    for _ in range(3):
        for y in outs:
            y.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        # compare link by link: reference of entry i is computed from the DEVICE output of entry i-1
        x_prev = None
        for i, ((n_out, k_in), y) in enumerate(zip(shapes, outs)):
            yy = y.cpu().numpy()
            assert np.isfinite(yy).all(), i
            if i == 0:
                assert_close(yy, refs[0])
            else:
                e = seq.keep[i]
                w_dec = oracle.np_decompress(e[1].cpu().numpy(), e[2].cpu().numpy(), e[3].cpu().numpy())
                ob = None if e[5] is None else e[5].cpu().numpy()
                assert_close(yy, oracle.np_linear(x_prev, w_dec, ob), i)
            x_prev = yy


def test_gemv_sequence_results_passed_on_in_parts(hip, device, oracle):
    """Batch 1, streaming layout, every dependency carried by data: the launch runs on the data-flow
    kernel, where an entry that a later entry reads and that has four row blocks or more in a
    workgroup publishes its results two row blocks at a time.  The producers here have several
    pieces of x per wave (k_in 8192), five row blocks in every workgroup (20480 rows: passes of 2,
    2, 1) and five in some workgroups and four in the others (16896 rows); every link of the chain
    is checked against the oracle applied to what the device fed it."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    shapes = [(16384, 8192), (1024, 16384), (20480, 1024), (512, 20480), (4096, 512), (16896, 4096), (256, 16896)]
    seq, refs, _ = _sequence_case(hip, device, oracle, shapes, 1, chained=True, seed=77)
    acts = [None, None, "gelu_tanh", None, None, "relu", None]  # (on two of the entries that publish in parts)
    flow, outs = GemvSequence(device), []
    for i, (x, packed, scale, bias, y, ob) in enumerate(seq.keep):
        y2 = torch.full_like(y, float("nan"))
        flow.add(outs[-1] if i > 0 else x, prepack_gemv(packed, scale, bias), None, None, y2, ob, wait_previous=i > 0,
                 activation=acts[i])
        outs.append(y2)
    for _ in range(3):
        for y in outs:
            y.fill_(float("nan"))
        flow.run()
        torch.cuda.synchronize()
        assert int(flow.status.item()) == 0
        x_prev = None
        for i, y in enumerate(outs):
            yy = y.cpu().numpy()
            assert np.isfinite(yy).all(), i
            if i == 0:
                assert_close(yy, refs[0])
            else:
                e = seq.keep[i]
                w_dec = oracle.np_decompress(e[1].cpu().numpy(), e[2].cpu().numpy(), e[3].cpu().numpy())
                assert_close(yy, oracle.np_linear(x_prev, w_dec, None if e[5] is None else e[5].cpu().numpy(), acts[i]), i)
            x_prev = yy


@pytest.mark.parametrize("streaming", [False, True])
@pytest.mark.parametrize("hidden,ffn,inside", [(1024, 4096, 0), (1024, 4096, 1536), (4096, 16384, 0)])
def test_gemv_sequence_x_from_several_producers(hip, device, oracle, streaming, hidden, ffn, inside):
    """Batch 1: an entry whose x is the results of TWO earlier entries that lie end to end in memory
    (the `up` projection's and the first third of a v|q|k projection's: the attention output and the
    second feed-forward layer of a parallel decoder block as one product over [up | v]).  It starts
    `inside` values into the first producer's results.  Two layers, the second reading the first's
    output; every entry is checked against the oracle applied to what the device fed it."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    seq, checks = GemvSequence(device), []
    x = to_dev(activations(1, hidden, 3), device)

    def entry(x_in, n_out, y, activation=None):
        k_in = x_in.shape[1]
        packed, scale, bias, w_dec = _full_size_weight(oracle, n_out, k_in, 7000 + 10 * (hidden + inside) + len(checks))
        dev = tuple(to_dev(a, device) for a in (packed, scale, bias))
        if streaming:
            seq.add(x_in, prepack_gemv(*dev), None, None, y, activation=activation)
        else:
            seq.add(x_in, *dev, y, activation=activation)
        checks.append((x_in, w_dec, y, activation))

    outs = []
    for layer in range(2):
        both = torch.full((1, ffn + 3 * hidden), float("nan"), dtype=torch.float16, device=device)
        y = torch.full((1, hidden), float("nan"), dtype=torch.float16, device=device)
        entry(x, ffn, both[:, :ffn], "gelu_tanh")
        entry(x, 3 * hidden, both[:, ffn:])
        entry(both[:, inside:ffn + hidden], hidden, y)
        outs += [both, y]
        x = y
    for _ in range(3):
        for t in outs:
            t.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        for i, (x_in, w_dec, y, activation) in enumerate(checks):
            yy = y.cpu().numpy()
            assert np.isfinite(yy).all(), i
            assert_close(yy, oracle.np_linear(x_in.cpu().numpy(), w_dec, None, activation), i)



def test_gemv_sequence_two_entries_per_layer(hip, device, oracle):
    """The decoder block as two entries: up, v, q and k stacked into one 28672 x 4096 entry (seven row
    blocks per workgroup, passed on in parts of 2, 2, 2 and 1), then the joint output product over the
    first 20480 of its results.  Two layers, streaming layout, batch 1; every entry against the oracle
    applied to what the device fed it."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    hidden, ffn = 4096, 16384
    seq, checks = GemvSequence(device), []
    x = to_dev(activations(1, hidden, 4), device)
    for layer in range(2):
        first = torch.full((1, ffn + 3 * hidden), float("nan"), dtype=torch.float16, device=device)
        y = torch.full((1, hidden), float("nan"), dtype=torch.float16, device=device)
        for x_in, n_out, out, activation in ((x, ffn + 3 * hidden, first, "relu"), (first[:, : ffn + hidden], hidden, y, None)):
            packed, scale, bias, w_dec = _full_size_weight(oracle, n_out, x_in.shape[1], 8000 + len(checks))
            seq.add(x_in, prepack_gemv(*(to_dev(a, device) for a in (packed, scale, bias))), None, None, out, activation=activation)
            checks.append((x_in, w_dec, out, activation))
        x = y
    for _ in range(3):
        for _, _, out, _ in checks:
            out.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        for i, (x_in, w_dec, out, activation) in enumerate(checks):
            assert_close(out.cpu().numpy(), oracle.np_linear(x_in.cpu().numpy(), w_dec, None, activation), i)

@pytest.mark.parametrize("m_rows,chained", [(1, False), (2, False), (4, False), (1, True), (4, True)])
def test_gemv_sequence_streaming_layout(hip, device, oracle, m_rows, chained):
    """Weights in the streaming layout of gq_gemv_prepack_f16 give what the same sequence gives on
    the three variables, with ragged row counts, waits, and both layouts mixed in one sequence.
    Another kernel runs them when the whole launch is in the streaming layout (fp32 sums taken in
    another order): the two agree to a few fp16 roundings, not bit for bit; a chain of entries
    carries the difference of its inputs along."""
    from popxl_addons._gq_hip import GemvSequence, GQHipError, prepack_gemv

    if chained:
        shapes = [(4096, 4096), (2048, 4096), (4096, 2048), (16384, 4096), (4096, 16384), (520, 4096)]
    else:
        shapes = [(4096, 4096), (1000, 4096), (16384, 4096), (4096, 16384), (16, 512), (5000, 1536), (40, 8192)]
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, m_rows, chained=chained)
    for mixed in (False, True):
        seq2, outs2 = GemvSequence(device), []
        for i, (x, packed, scale, bias, y, ob) in enumerate(seq.keep):
            y2 = torch.full_like(y, float("nan"))
            x2 = outs2[-1] if chained and i > 0 else x
            if mixed and i % 3 == 1:
                seq2.add(x2, packed, scale, bias, y2, ob, wait_previous=chained and i > 0)
            else:
                w = prepack_gemv(packed, scale, bias)
                assert w.blob.numel() == int(-(-packed.shape[0] // 16) * 16 * x.shape[1] * 0.5625)
                seq2.add(x2, w, None, None, y2, ob, wait_previous=chained and i > 0)
            outs2.append(y2)
        for _ in range(2):
            for y in outs + outs2:
                y.fill_(float("nan"))
            seq.run()
            seq2.run()
            torch.cuda.synchronize()
            assert int(seq.status.item()) == 0 and int(seq2.status.item()) == 0
            for i, (y, y2) in enumerate(zip(outs, outs2)):
                assert torch.isfinite(y2).all(), i
                top = y.float().abs().max().item()
                worst = (y.float() - y2.float()).abs().max().item()
                assert worst <= (4e-3 if chained else 1.5e-3) * top, (i, mixed, worst / top)
        if not chained:
            for y2, ref in zip(outs2, refs):
                assert_close(y2.cpu().numpy(), ref)
    # a blob next to an entry that only the per-entry kernels can run (group 32): the sequence executes in
    # runs -- the blob's entry on the persistent kernel, the other as a launch of its own
    rng = np.random.default_rng(4)
    w32 = rng.normal(0, 0.02, (96, 256)).astype(np.float16)
    p32, s32, b32 = group_quantize_compress_numpy(w32, 32)
    mixed_seq = GemvSequence(device)
    x, packed, scale, bias, y, ob = seq.keep[0]
    want = y.clone()
    y.fill_(float("nan"))
    mixed_seq.add(x, prepack_gemv(packed, scale, bias), None, None, y, ob)
    x32 = activations(m_rows, 256, 1)
    y32 = torch.full((m_rows, 96), float("nan"), dtype=torch.float16, device=device)
    mixed_seq.add(to_dev(x32, device), *(to_dev(a, device) for a in (p32, s32, b32)), y32)
    mixed_seq.run()
    mixed_seq.check()
    top = want.float().abs().max().item()
    assert (y.float() - want.float()).abs().max().item() <= 1.5e-3 * top
    assert_close(y32.cpu().numpy(), oracle.np_linear(x32, oracle.np_decompress(p32, s32, b32)))
    # more than four batch rows: outside the persistent kernels, the blob's entry is a launch of the one-shot kernel,
    # which reads the streaming layout as well; what stays refused is more than sixteen
    w_dec = oracle.np_decompress(*(a.cpu().numpy() for a in (packed, scale, bias)))
    for rows in (5, 16):
        tall = GemvSequence(device)
        x_tall = activations(rows, x.shape[1], 2)
        y_tall = torch.full((rows, packed.shape[0]), float("nan"), dtype=torch.float16, device=device)
        tall.add(to_dev(x_tall, device), prepack_gemv(packed, scale, bias), None, None, y_tall, ob)
        tall.run()
        tall.check()
        assert_close(y_tall.cpu().numpy(), oracle.np_linear(x_tall, w_dec, None if ob is None else ob.cpu().numpy()), rows)
    too_tall = GemvSequence(device)
    x17 = to_dev(activations(17, x.shape[1], 2), device)
    too_tall.add(x17, prepack_gemv(packed, scale, bias), None, None, torch.empty((17, packed.shape[0]), dtype=torch.float16, device=device))
    with pytest.raises(GQHipError) as e:
        too_tall.run()
    assert "streaming layout" in str(e.value)


@pytest.mark.parametrize("seed", range(8))
def test_gemv_sequence_random_graphs(hip, device, oracle, seed):
    """Seeded random sequences: shapes with ragged row counts and 1 - 16 chunks, batch 1 - 4, each
    entry reading the activations or the output of a random earlier entry (and waiting for it),
    random epilogues, both weight layouts mixed.  Every entry is checked against the oracle applied
    to the input the device actually had."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    rng = np.random.default_rng(1000 + seed)
    m_rows = int(rng.integers(1, 5))
    widths = [512 * int(rng.integers(1, 5)) for _ in range(3)] + [512 * int(rng.integers(5, 17))]
    n_entries = int(rng.integers(6, 15))
    x0 = activations(m_rows, widths[0], seed)
    seq = GemvSequence(device)
    feeds = [(to_dev(x0, device), widths[0], None)]  # (device tensor, width, producing entry)
    entries = []
    for i in range(n_entries):
        x_dev, k_in, producer = feeds[int(rng.integers(0, len(feeds)))]
        n_out = int(rng.choice(widths)) if rng.random() < 0.6 else int(rng.integers(1, 1500))
        w = rng.normal(0, 1.0 / np.sqrt(k_in), (n_out, k_in)).astype(np.float16)
        packed, scale, bias = group_quantize_compress_numpy(w, 64)
        ob = rng.normal(0, 0.1, (n_out,)).astype(np.float16) if rng.random() < 0.5 else None
        act = [None, "relu", "gelu_tanh"][int(rng.integers(0, 3))]
        pd, sd, bd = (to_dev(a, device) for a in (packed, scale, bias))
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        args = (prepack_gemv(pd, sd, bd), None, None) if rng.random() < 0.5 else (pd, sd, bd)
        seq.add(x_dev, *args, y, None if ob is None else to_dev(ob, device), wait_for=producer, activation=act)
        entries.append((x_dev, y, oracle.np_decompress(packed, scale, bias), ob, act))
        if n_out % 512 == 0:
            feeds.append((y, n_out, i))
    for _ in range(2):
        for _x, y, *_rest in entries:
            y.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        for i, (x_dev, y, w_dec, ob, act) in enumerate(entries):
            got = y.cpu().numpy()
            assert np.isfinite(got).all(), (seed, i)
            assert_close(got, oracle.np_linear(x_dev.cpu().numpy(), w_dec, ob, act), (seed, i))


@pytest.mark.parametrize("seed", range(16))
def test_gemv_sequence_random_graphs_with_reused_buffers(hip, device, seed):
    """Seeded random sequences in which outputs OVERWRITE buffers that earlier entries read or wrote
    (what a model with one buffer per role does), declared as the interface asks: an entry waits for the
    last entry that wrote its x and for the last entry that read or wrote the buffer it overwrites.
    The host's plan of a launch has to tell exchanges from reported completion for every such case.
    Checked against the same entries run one call at a time, in order, on a second set of buffers with
    the same initial contents (the arithmetic of an entry is held to the oracle by the other tests;
    this one holds the ORDER): every buffer ends with the values the in-order run leaves."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    rng = np.random.default_rng(7000 + seed)
    m_rows = int(rng.integers(1, 5))
    widths = sorted({512 * int(rng.integers(1, 9)) for _ in range(3)})
    n_entries = int(rng.integers(8, 20))
    # two universes of buffers with the same contents: [0] the sequence's, [1] the in-order run's
    buffers = []  # (width, [tensor, tensor])

    def new_buffer(width, fill=None):
        t = torch.full((m_rows, width), float("nan"), dtype=torch.float16, device=device) if fill is None else to_dev(fill, device)
        buffers.append((width, [t, t.clone()]))
        return len(buffers) - 1

    for w in widths:
        new_buffer(w, activations(m_rows, w, seed + w))
    written = {i for i in range(len(buffers))}  # buffers that hold numbers
    last_touch = {}  # buffer -> index of the last entry that read or wrote it
    last_write = {}
    seq = GemvSequence(device)
    plan = []
    for i in range(n_entries):
        x_id = int(rng.choice(sorted(written)))
        k_in = buffers[x_id][0]
        n_out = int(rng.choice(widths))
        candidates = [b for b, (w, _) in enumerate(buffers) if w == n_out and b != x_id and b >= len(widths)]
        y_id = int(rng.choice(candidates)) if candidates and rng.random() < 0.5 else new_buffer(n_out)
        w = rng.normal(0, 1.0 / np.sqrt(k_in), (n_out, k_in)).astype(np.float16)
        pd, sd, bd = (to_dev(a, device) for a in group_quantize_compress_numpy(w, 64))
        act = [None, "relu", "gelu_tanh"][int(rng.integers(0, 3))]
        waits = [last_write.get(x_id), last_touch.get(y_id)]
        waits = [v for v in waits if v is not None]
        args = (prepack_gemv(pd, sd, bd), None, None) if rng.random() < 0.5 else (pd, sd, bd)
        seq.add(buffers[x_id][1][0], *args, buffers[y_id][1][0], None, wait_for=max(waits) if waits else None, activation=act)
        plan.append((x_id, y_id, (pd, sd, bd), n_out, k_in, act))
        last_touch[x_id] = i
        last_touch[y_id] = i
        last_write[y_id] = i
        written.add(y_id)
    # the in-order run
    stream = torch.cuda.current_stream().cuda_stream
    for x_id, y_id, (pd, sd, bd), n_out, k_in, act in plan:
        x, y = buffers[x_id][1][1], buffers[y_id][1][1]
        hip.call("gq_linear_act_f16", x.data_ptr(), m_rows, pd.data_ptr(), sd.data_ptr(), bd.data_ptr(), 0, y.data_ptr(), n_out, k_in,
                 64, hip.activation_code(act), stream)
    torch.cuda.synchronize()
    initial = [t[0].clone() for _, t in buffers]
    for run in range(2):
        for (_, t), first in zip(buffers, initial):
            t[0].copy_(first)
        seq.run()
        seq.check()
        for b, (_, (got, want)) in enumerate(buffers):
            if b not in written:
                continue
            g, w_ = got.float().cpu().numpy(), want.float().cpu().numpy()
            assert np.isfinite(g).all(), (seed, run, b)
            assert np.abs(g - w_).max() <= 5e-3 * max(np.abs(w_).max(), 1e-3), (seed, run, b, np.abs(g - w_).max(), np.abs(w_).max())


def test_gemv_sequence_fallback_and_graph(hip, device, oracle):
    """Shapes outside the persistent kernel (group 32) run entry by entry; the persistent kernel
    replays correctly from a captured graph."""
    from popxl_addons._gq_hip import GemvSequence

    rng = np.random.default_rng(3)
    seq = GemvSequence(device)
    w = rng.normal(0, 0.02, (96, 256)).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, 32)
    x = activations(2, 256, 1)
    y = torch.empty((2, 96), dtype=torch.float16, device=device)
    seq.add(to_dev(x, device), to_dev(packed, device), to_dev(scale, device), to_dev(bias, device), y)
    seq.run()
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.np_linear(x, oracle.np_decompress(packed, scale, bias)))

    shapes = [(4096, 4096), (4096, 4096), (1024, 4096)]
    seq2, refs, outs = _sequence_case(hip, device, oracle, shapes, 1, chained=True, seed=60)
    seq2.run()
    torch.cuda.synchronize()
    want = [o.clone() for o in outs]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        seq2.run()
    for _ in range(3):
        for o in outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert int(seq2.status.item()) == 0
        for o, w_ in zip(outs, want):
            assert torch.equal(o, w_)


@pytest.mark.parametrize("m_rows", [1, 3])
def test_gemv_sequence_wait_for_earlier_entry(hip, device, oracle, m_rows):
    """Declared dependencies (`wait_entries`): two layers of a parallel decoder block.  q, k, v and
    up read the layer input; o waits for v only (up keeps streaming meanwhile), down waits for up,
    and the next layer's projections wait for everything.  Every output equals the single-call
    GEMV on the same device inputs, bit for bit or within tolerance of the oracle."""
    from popxl_addons._gq_hip import GemvSequence

    hidden, ffn = 1024, 4096
    rng = np.random.default_rng(77)
    seq = GemvSequence(device)

    def weight(n_out, k_in):
        w = rng.normal(0, 1.0 / np.sqrt(k_in), (n_out, k_in)).astype(np.float16)
        return tuple(to_dev(a, device) for a in group_quantize_compress_numpy(w, 64))

    def out(n):
        return torch.full((m_rows, n), float("nan"), dtype=torch.float16, device=device)

    x = to_dev(activations(m_rows, hidden, 5), device)
    plan = []  # (entry index, x tensor, weights, y tensor)
    last = None
    for layer in range(2):
        ys = {name: out(hidden) for name in ("q", "k", "v", "o", "down")}
        ys["up"] = out(ffn)
        idx = {}
        for name in ("q", "k", "v", "up"):
            w = weight(ffn if name == "up" else hidden, hidden)
            idx[name] = seq.add(x, *w, ys[name], wait_for=last if name == "q" else None)
            plan.append((idx[name], x, w, ys[name]))
        w = weight(hidden, hidden)
        idx["o"] = seq.add(ys["v"], *w, ys["o"], wait_for=idx["v"])
        plan.append((idx["o"], ys["v"], w, ys["o"]))
        w = weight(hidden, ffn)
        idx["down"] = seq.add(ys["up"], *w, ys["down"], wait_for=idx["up"])
        plan.append((idx["down"], ys["up"], w, ys["down"]))
        x, last = ys["down"], idx["down"]  # next layer reads `down`; waiting for it covers o as well
    with pytest.raises(ValueError):
        seq.add(x, *weight(hidden, hidden), out(hidden), wait_for=len(seq.entries))  # cannot wait for itself

    for _ in range(3):
        for _, _, _, y in plan:
            y.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        for i, x_in, (p, s, b), y in plan:
            single = torch.empty_like(y)
            hip.call("gq_gemv_f16", x_in.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0,
                     single.data_ptr(), y.shape[1], x_in.shape[1], 64, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            yy, ss = y.cpu().numpy(), single.cpu().numpy()
            assert np.isfinite(yy).all(), i
            assert normalised_error(yy, ss.astype(np.float32)) <= 2e-3, i  # same inputs, other summation order
            w_dec = oracle.np_decompress(p.cpu().numpy(), s.cpu().numpy(), b.cpu().numpy())
            assert_close(yy, oracle.np_linear(x_in.cpu().numpy(), w_dec, None), i)


def test_gemv_sequence_longer_than_one_launch(hip, device, oracle):
    """More entries than one launch of the persistent kernel holds (128): the sequence continues
    in a second launch, and dependencies that reach back across the boundary hold."""
    from popxl_addons._gq_hip import GemvSequence

    rng = np.random.default_rng(21)
    seq = GemvSequence(device)
    n_entries, width = 140, 512
    x0 = activations(2, width, 9)
    weights, outs = [], []
    x_in = to_dev(x0, device)
    for i in range(n_entries):
        w = rng.normal(0, 1.0 / np.sqrt(width), (width, width)).astype(np.float16)
        packed, scale, bias = group_quantize_compress_numpy(w, 64)
        y = torch.full((2, width), float("nan"), dtype=torch.float16, device=device)
        # every third entry starts a new chain from x0; the others read their predecessor
        chained = i % 3 != 0
        seq.add(x_in if chained else to_dev(x0, device), to_dev(packed, device), to_dev(scale, device),
                to_dev(bias, device), y, wait_for=i - 1 if chained else None)
        weights.append((packed, scale, bias, chained))
        outs.append(y)
        x_in = y
    for _ in range(2):
        for y in outs:
            y.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        prev = None
        for i, ((packed, scale, bias, chained), y) in enumerate(zip(weights, outs)):
            yy = y.cpu().numpy()
            assert np.isfinite(yy).all(), i
            x_host = prev if chained else x0
            assert_close(yy, oracle.np_linear(x_host, oracle.np_decompress(packed, scale, bias), None), i)
            prev = yy


@pytest.mark.parametrize("activation,code", [("relu", 1), ("gelu_tanh", 2)])
@pytest.mark.parametrize("m_rows", [1, 8, 40, 300])
def test_fused_activation_epilogue(hip, device, oracle, activation, code, m_rows):
    """gq_linear_act_f16: the activation is applied to sum + out_bias in every kernel the dispatch
    reaches (MFMA GEMV, generic GEMV, single GEMV through the persistent kernel, pipelined GEMM,
    tile GEMM)."""
    shapes = ((520, 1024, 64), (96, 192, 64), (24, 40, 20)) + (((8192, 4096, 64),) if m_rows == 1 else ())
    for n_out, k_in, gs in shapes:
        x, packed, scale, bias, ob, _ = _case(oracle, n_out, k_in, gs, m_rows, 71, True)
        y_ref = oracle.np_linear(x, oracle.np_decompress(packed, scale, bias), ob, activation)
        xd, pd, sd, bd, od = (to_dev(a, device) for a in (x, packed, scale, bias, ob))
        y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
        hip.call("gq_linear_act_f16", xd.data_ptr(), m_rows, pd.data_ptr(), sd.data_ptr(), bd.data_ptr(), od.data_ptr(),
                 y.data_ptr(), n_out, k_in, gs, code, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        yy = y.cpu().numpy()
        assert np.isfinite(yy).all()
        assert_close(yy, y_ref, (n_out, k_in, gs))
        if activation == "relu":
            assert (yy >= 0).all()


@pytest.mark.parametrize("m_rows", [1, 4, 8])
def test_gemv_sequence_activation(hip, device, oracle, m_rows):
    """Per-entry activation in a sequence: up-projection with GELU feeding the down-projection
    (persistent kernel for m_rows <= 4, one launch per entry above)."""
    from popxl_addons._gq_hip import GemvSequence

    hidden, ffn = 512, 2048
    rng = np.random.default_rng(91)
    x = activations(m_rows, hidden, 3)
    w_up = rng.normal(0, 1.0 / np.sqrt(hidden), (ffn, hidden)).astype(np.float16)
    w_down = rng.normal(0, 1.0 / np.sqrt(ffn), (hidden, ffn)).astype(np.float16)
    b_up = rng.normal(0, 0.5, (ffn,)).astype(np.float16)
    up = group_quantize_compress_numpy(w_up, 64)
    down = group_quantize_compress_numpy(w_down, 64)
    seq = GemvSequence(device)
    y_up = torch.full((m_rows, ffn), float("nan"), dtype=torch.float16, device=device)
    y_down = torch.full((m_rows, hidden), float("nan"), dtype=torch.float16, device=device)
    first = seq.add(to_dev(x, device), *(to_dev(a, device) for a in up), y_up, to_dev(b_up, device), activation="gelu_tanh")
    seq.add(y_up, *(to_dev(a, device) for a in down), y_down, wait_for=first, activation="relu")
    for _ in range(2):
        y_up.fill_(float("nan"))
        y_down.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert int(seq.status.item()) == 0
        got_up, got_down = y_up.cpu().numpy(), y_down.cpu().numpy()
        assert_close(got_up, oracle.np_linear(x, oracle.np_decompress(*up), b_up, "gelu_tanh"))
        assert_close(got_down, oracle.np_linear(got_up, oracle.np_decompress(*down), None, "relu"))


def test_gemv_sequence_gives_up_and_recovers(hip, device, oracle):
    """A poller that sees no progress for `spin_limit` polls gives up: the kernel sets *status and
    drains with every workgroup exiting normally.  With a limit of one poll a chained sequence
    cannot finish its waits; afterwards the same sequence with the default limit is correct, i.e.
    the progress words were left at zero."""
    from popxl_addons._gq_hip import GemvSequence, GQHipError

    shapes = [(4096, 4096), (16384, 4096), (4096, 16384), (4096, 4096)]
    impatient = GemvSequence(device, spin_limit=1)
    patient = GemvSequence(device, own_workspace=True)
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, 1, chained=True, seed=70)
    for s2 in (impatient, patient):
        for i, (x, packed, scale, bias, y, ob) in enumerate(seq.keep):
            s2.add(x, packed, scale, bias, y, ob, wait_previous=i > 0)
    impatient._finalise()
    patient._finalise()
    patient._workspace = impatient._workspace  # the same progress words, one run after the other
    impatient.run()
    torch.cuda.synchronize()
    assert int(impatient.status.item()) == 1
    with pytest.raises(GQHipError):
        impatient.check()
    control = (256 + 2) * 128  # bytes: the workgroups' progress lines, the announcement, the exit count
    assert not impatient._workspace[:control].any(), "progress words must be back at zero after a run that gave up"
    for _ in range(2):
        for y in outs:
            y.fill_(float("nan"))
        patient.run()
        patient.check()
        x_prev = None
        for i, y in enumerate(outs):
            yy = y.cpu().numpy()
            if i == 0:
                assert_close(yy, refs[0])
            else:
                e = seq.keep[i]
                w_dec = oracle.np_decompress(e[1].cpu().numpy(), e[2].cpu().numpy(), e[3].cpu().numpy())
                assert_close(yy, oracle.np_linear(x_prev, w_dec, None if e[5] is None else e[5].cpu().numpy()), i)
            x_prev = yy


def test_gemv_sequences_with_own_workspaces_on_two_streams(hip, device, oracle):
    """Two chained sequences, each with progress words of its own, enqueued in turn on two streams
    that are ordered by events (the persistent kernel needs the whole device: two of them must not
    run at the same time): both are correct."""
    from popxl_addons._gq_hip import GemvSequence

    shapes = [(4096, 4096), (2048, 4096), (4096, 2048), (4096, 4096)]
    cases = []
    for seed in (80, 90):
        seq, refs, outs = _sequence_case(hip, device, oracle, shapes, 2, chained=True, seed=seed)
        own = GemvSequence(device, own_workspace=True)
        for i, (x, packed, scale, bias, y, ob) in enumerate(seq.keep):
            own.add(x, packed, scale, bias, y, ob, wait_previous=i > 0)
        cases.append((own, seq, refs, outs))
    streams = [torch.cuda.Stream(device=device) for _ in cases]
    torch.cuda.synchronize()
    for _ in range(3):
        for (own, _, _, outs), stream, other in zip(cases, streams, reversed(streams)):
            stream.wait_stream(other)
            with torch.cuda.stream(stream):
                own.run()
        torch.cuda.synchronize()
    for own, seq, refs, outs in cases:
        own.check()
        x_prev = None
        for i, y in enumerate(outs):
            yy = y.cpu().numpy()
            if i == 0:
                assert_close(yy, refs[0])
            else:
                e = seq.keep[i]
                w_dec = oracle.np_decompress(e[1].cpu().numpy(), e[2].cpu().numpy(), e[3].cpu().numpy())
                assert_close(yy, oracle.np_linear(x_prev, w_dec, None if e[5] is None else e[5].cpu().numpy()), i)
            x_prev = yy


@pytest.mark.parametrize("next_input", ["o", "alternate"])
@pytest.mark.parametrize("m_rows", [1, 4])
def test_gemv_sequence_decoder_schedule_at_full_size(hip, device, oracle, m_rows, next_input):
    """The schedule the layer-stack benchmark times, on three full-size layers with real data flowing
    through every declared wait: per layer the entries up (16384 x 4096, waits for the previous
    layer), fused qkv (12288 x 4096), down (4096 x 16384, waits for up), o (4096 x 4096, waits for
    qkv), every weight in the streaming layout.  up and qkv read the layer input, down reads up's
    output, o reads 4096-wide rows out of qkv's output, and the next layer's input is o's output
    ("o": what the benchmark times; every result then travels through the kernel's tagged exchange)
    or o's and down's in turn ("alternate": the entries that read down's output wait for more than
    its producer, so they wait for reported completion, next to entries that use the exchange).
    Every entry is checked against the oracle applied to the
    inputs the device had; then the same sequence with the buffers of a role shared by all layers
    (as the benchmark does: write-after-read hazards that only the declared waits resolve) must
    end with the same bits."""
    from popxl_addons._gq_hip import GemvSequence, prepack_gemv

    hidden, ffn, n_layers = 4096, 16384, 3

    def weight(n_out, k_in, seed):
        packed, scale, bias, w_dec = _full_size_weight(oracle, n_out, k_in, seed)  # (the same for every case of this test)
        return w_dec, prepack_gemv(*(to_dev(a, device) for a in (packed, scale, bias)))

    def out(n):
        return torch.full((m_rows, n), float("nan"), dtype=torch.float16, device=device)

    def v_rows(y_qkv):  # m_rows x 4096 contiguous values out of qkv's output, starting at its column 8192
        return y_qkv.view(-1)[2 * hidden : 2 * hidden + m_rows * hidden].view(m_rows, hidden)

    weights = [{name: weight(*shape, 500 + 10 * layer + i)
                for i, (name, shape) in enumerate((("up", (ffn, hidden)), ("qkv", (3 * hidden, hidden)),
                                                   ("down", (hidden, ffn)), ("o", (hidden, hidden))))} for layer in range(n_layers)]
    h0 = to_dev(activations(m_rows, hidden, 9), device)

    def build(shared_buffers):
        seq, plan = GemvSequence(device), []
        # shared: one up and one qkv buffer for all layers; o and down, which carry the layer input
        # over to the next layer, alternate between two buffers (down of layer L + 1 does not wait
        # for qkv of layer L + 1, which may still be reading down of layer L)
        shared = [{"up": None, "qkv": None, "down": out(hidden), "o": out(hidden)} for _ in range(2)]
        shared[0]["up"] = shared[1]["up"] = out(ffn)
        shared[0]["qkv"] = shared[1]["qkv"] = out(3 * hidden)
        h, last = h0, None
        for layer in range(n_layers):
            ys = shared[layer % 2] if shared_buffers else {"up": out(ffn), "qkv": out(3 * hidden), "down": out(hidden), "o": out(hidden)}
            w = weights[layer]
            up = seq.add(h, w["up"][1], None, None, ys["up"], wait_for=last)
            qkv = seq.add(h, w["qkv"][1], None, None, ys["qkv"])
            seq.add(ys["up"], w["down"][1], None, None, ys["down"], wait_for=up)
            last = seq.add(v_rows(ys["qkv"]), w["o"][1], None, None, ys["o"], wait_for=qkv)
            plan += [(h, w["up"][0], ys["up"]), (h, w["qkv"][0], ys["qkv"]), (ys["up"], w["down"][0], ys["down"]),
                     (v_rows(ys["qkv"]), w["o"][0], ys["o"])]
            h = ys["o"] if layer % 2 == 0 or next_input == "o" else ys["down"]
        return seq, plan

    seq, plan = build(shared_buffers=False)
    assert [e[10] for e in seq.entries] == [0, 0, 1, 2, 4, 0, 5, 6, 8, 0, 9, 10]
    for run in range(2):
        for _, _, y in plan:
            y.fill_(float("nan"))
        seq.run()
        seq.check()
        for i, (x_in, w_dec, y) in enumerate(plan):
            assert_close(y.cpu().numpy(), oracle.np_linear(x_in.cpu().numpy(), w_dec, None), (run, i))
    final = [y.clone() for _, _, y in plan[-4:]]
    shared_seq, shared_plan = build(shared_buffers=True)
    for run in range(2):
        for _, _, y in shared_plan[-4:]:
            y.fill_(float("nan"))
        shared_seq.run()
        shared_seq.check()
        for want, (_, _, y) in zip(final, shared_plan[-4:]):
            assert torch.equal(want, y), run


# --------------------------------------------------------------------------------------------------
# the benchmark's own 28-layer schedules, and what happens when a sequence cannot finish


def test_benchmark_stack_28_layers_against_oracle(hip, device, oracle):
    """The exact 28-layer schedules that bench.py times at one batch row (four entries per layer and
    two entries per layer, every weight in the streaming layout, 3.17 GB of packed weights): after the
    passes, the last layer's outputs equal the oracle's linear over the oracle-decompressed weights,
    applied to the inputs the device had -- 27 layers of ring wrap-around, result exchange and
    launches of 112 / 56 entries lie in front of them.  bench.py does the comparison when it is
    handed the oracle (it raises if the error exceeds 1e-2 or the kernel gave up)."""
    import bench

    modes = ("sequence_decoder_data_flow_streaming_layout", "sequence_decoder_data_flow_two_entries_streaming_layout",
             "sequence_parallel_block_fused_qkv_ffn_first_streaming_layout")
    r = bench.bench_stack(hip, device, 1, passes=3, warmup=1, modes=modes, oracle=oracle)
    for mode in modes:
        assert r[mode]["status"] == 0
        assert r[mode]["max_error_vs_oracle"] <= REGRESSION_TOL, (mode, r[mode])
        assert r[mode]["max_error_vs_single_call"] <= REGRESSION_TOL, (mode, r[mode])
    torch.cuda.empty_cache()


def test_benchmark_stack_28_layers_batch_4_against_oracle(hip, device, oracle):
    """The same at four batch rows (the LDS-ring kernel)."""
    import bench

    modes = ("sequence_decoder_data_flow_streaming_layout",)
    r = bench.bench_stack(hip, device, 4, passes=2, warmup=1, modes=modes, oracle=oracle)
    assert r[modes[0]]["status"] == 0 and r[modes[0]]["max_error_vs_oracle"] <= REGRESSION_TOL, r[modes[0]]
    torch.cuda.empty_cache()


def test_benchmark_stack_28_layers_batch_8_against_oracle(hip, device, oracle):
    """Eight batch rows, which the persistent kernels do not take: the two launches per layer through the
    layer's entry point (the one-shot kernel on the weights' streaming-layout copies), as bench.py times them."""
    import bench

    modes = ("streaming_layout_two_entries_graph",)
    r = bench.bench_stack(hip, device, 8, passes=2, warmup=1, modes=modes, oracle=oracle)
    assert r[modes[0]]["max_error_vs_oracle"] <= REGRESSION_TOL and r[modes[0]]["max_error_vs_single_call"] <= REGRESSION_TOL, r[modes[0]]
    torch.cuda.empty_cache()


def _chained_streaming_case(hip, device, oracle, shapes, seed):
    """Chained entries at one batch row, every weight in the streaming layout: (entries, oracle results)."""
    from popxl_addons._gq_hip import prepack_gemv

    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, 1, chained=True, seed=seed)
    entries = [(x, prepack_gemv(packed, scale, bias), y, ob) for x, packed, scale, bias, y, ob in seq.keep]
    return entries, seq, refs, outs


def _assert_chain(oracle, seq, refs, outs):
    x_prev = None
    for i, y in enumerate(outs):
        yy = y.cpu().numpy()
        if i == 0:
            assert_close(yy, refs[0])
        else:
            e = seq.keep[i]
            w_dec = oracle.np_decompress(e[1].cpu().numpy(), e[2].cpu().numpy(), e[3].cpu().numpy())
            assert_close(yy, oracle.np_linear(x_prev, w_dec, None if e[5] is None else e[5].cpu().numpy()), i)
        x_prev = yy


# word index of the data-flow kernel's launch count in a sequence workspace: 256 progress lines, the
# announcement, the exit count and the epoch (a 128-byte line each), rounded up to 256 bytes, then the
# 16 MiB exchange of the other kernel
_FLOW_EPOCH_WORD = ((256 + 3) * 32 + 32 + 63) // 64 * 64 + (16 << 20) // 4


def test_data_flow_kernel_gives_up_and_recovers(hip, device, oracle):
    """The give-up path of the data-flow kernel (batch 1, streaming layout, every dependency carried by
    data): with a limit of one poll, a wave whose x has not arrived gives up at once, the kernel sets
    *status and every workgroup exits; the same entries on the same workspace with the default limit
    are then correct twice over, i.e. the halves of the exchange and the launch count were left
    consistent."""
    from popxl_addons._gq_hip import GemvSequence, GQHipError

    shapes = [(4096, 4096), (16384, 4096), (4096, 16384), (4096, 4096)]
    entries, seq, refs, outs = _chained_streaming_case(hip, device, oracle, shapes, seed=71)
    impatient = GemvSequence(device, spin_limit=1)
    patient = GemvSequence(device, own_workspace=True)
    for s2 in (impatient, patient):
        for i, (x, w, y, ob) in enumerate(entries):
            s2.add(x, w, None, None, y, ob, wait_previous=i > 0)
    impatient._finalise()
    patient._finalise()
    patient._workspace = impatient._workspace  # the same workspace, one run after the other
    words = impatient._workspace.view(torch.int32)
    assert int(words[_FLOW_EPOCH_WORD].item()) == 0
    impatient.run()
    torch.cuda.synchronize()
    assert int(impatient.status.item()) == 1
    assert int(words[_FLOW_EPOCH_WORD].item()) == 1, "the launch ran on the data-flow kernel and turned the exchange over"
    with pytest.raises(GQHipError):
        impatient.check()
    for run in range(2):
        for y in outs:
            y.fill_(float("nan"))
        patient.run()
        patient.check()
        assert int(words[_FLOW_EPOCH_WORD].item()) == run % 2
        _assert_chain(oracle, seq, refs, outs)


def test_gemv_sequence_run_raises_after_a_give_up(hip, device, oracle):
    """A run that gave up does not pass silently: the next run() of the object raises (it looks at the
    host copy of the status word that the earlier run left behind), once; after that the object
    works again."""
    from popxl_addons._gq_hip import GemvSequence, GQHipError

    shapes = [(4096, 4096), (2048, 4096), (4096, 2048)]
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, 2, chained=True, seed=72)
    impatient = GemvSequence(device, spin_limit=1)
    for i, (x, packed, scale, bias, y, ob) in enumerate(seq.keep):
        impatient.add(x, packed, scale, bias, y, ob, wait_previous=i > 0)
    impatient.run()
    torch.cuda.synchronize()
    assert int(impatient.status.item()) == 1
    with pytest.raises(GQHipError, match="gave up"):
        impatient.run()
    assert int(impatient.status.item()) == 0
    impatient.spin_limit = 0  # the default limit: the same entries, the same workspace
    for _ in range(2):
        for y in outs:
            y.fill_(float("nan"))
        impatient.run()
        impatient.check()
        _assert_chain(oracle, seq, refs, outs)


def test_gemv_sequence_second_stream_is_refused_while_the_first_is_busy(hip, device, oracle):
    """gq_gemv_sequence_f16 keeps its progress words in a block of the library, per device: a call on
    another stream while the first stream still has work pending is refused (GQ_ERR_UNSUPPORTED, nothing
    launched) instead of corrupting both; once the first stream has drained, the other stream may use
    the block."""
    from popxl_addons._gq_hip import GQ_ERR_UNSUPPORTED, GQHipError

    shapes = [(4096, 4096), (2048, 4096), (4096, 2048)]
    seq, refs, outs = _sequence_case(hip, device, oracle, shapes, 2, chained=True, seed=73)
    other = torch.cuda.Stream(device=device)
    a = torch.randn((8192, 8192), dtype=torch.float16, device=device)
    seq.run()  # (the first run copies the entries to the device, which waits for the stream)
    seq.check()
    for y in outs:
        y.fill_(float("nan"))
    torch.cuda.synchronize()
    for _ in range(40):  # tens of milliseconds of work on the current stream, then the sequence behind it
        a @ a
    seq.run()
    with torch.cuda.stream(other):
        with pytest.raises(GQHipError) as refused:
            seq.run()
    assert refused.value.code == GQ_ERR_UNSUPPORTED and "another stream" in str(refused.value)
    seq.check()
    _assert_chain(oracle, seq, refs, outs)
    for y in outs:
        y.fill_(float("nan"))
    torch.cuda.synchronize()  # (the fills are work of the first stream too)
    with torch.cuda.stream(other):  # the first stream is idle now
        seq.run()
    seq.check()
    _assert_chain(oracle, seq, refs, outs)
    seq.run()  # and back, after the other stream has drained
    seq.check()
