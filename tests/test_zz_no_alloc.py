"""gq_linear_kn_act_noalloc_f16: the fused matmul for weights grouped along the output features
with its scratch buffer (partial sums, arrival counters) in a device array of the library, for
callers that cannot allocate.  Checked through the C ABI against gq_linear_kn_act_f16 with a
caller-provided workspace, bit for bit, on calls in a row that share the array -- the later ones
smaller, so that they find the earlier ones' contents in it."""
import numpy as np
import pytest
import torch

from gq_testlib import activations, assert_bits_equal, to_dev
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy

pytestmark = pytest.mark.gpu


def _problem(device, k_in, n_out, gs, m_rows, seed):
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (k_in, n_out)).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, gs)
    out_bias = rng.normal(0, 1, (n_out,)).astype(np.float16)
    x = activations(m_rows, k_in, seed + 1)
    return tuple(to_dev(a, device) for a in (x, packed, scale, bias, out_bias))


def _with_workspace(hip, device, tensors, k_in, n_out, gs, m_rows, act):
    x, packed, scale, bias, out_bias = tensors
    need = hip.load().gq_linear_kn_workspace_bytes(m_rows, n_out, k_in, gs)
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=device)
    y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    hip.call("gq_linear_kn_act_f16", x.data_ptr(), m_rows, packed.data_ptr(), scale.data_ptr(), bias.data_ptr(),
             out_bias.data_ptr(), y.data_ptr(), n_out, k_in, gs, act, ws.data_ptr(), ws.numel(),
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return y.cpu().numpy(), need


def _no_alloc(hip, device, tensors, k_in, n_out, gs, m_rows, act):
    x, packed, scale, bias, out_bias = tensors
    y = torch.full((m_rows, n_out), float("nan"), dtype=torch.float16, device=device)
    import gc

    gc.collect()  # (tensors of earlier tests that are freed during the call would change the figures below)
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(device), torch.cuda.mem_get_info(device)[0]
    hip.call("gq_linear_kn_act_noalloc_f16", x.data_ptr(), m_rows, packed.data_ptr(), scale.data_ptr(), bias.data_ptr(),
             out_bias.data_ptr(), y.data_ptr(), n_out, k_in, gs, act, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    # neither through torch's allocator nor behind its back (device memory as the driver counts it)
    assert torch.cuda.memory_allocated(device) <= before
    assert torch.cuda.mem_get_info(device)[0] >= free_before
    return y.cpu().numpy()


def test_no_alloc_entry_point_matches_workspace_entry_point(hip, device):
    # (k_in, n_out, group, m_rows, activation): a large problem first, then smaller ones that reuse
    # the array with the first one's partial sums still in it, then a prefill batch (no scratch)
    calls = [(4096, 16384, 64, 4, 0), (4096, 4096, 64, 2, 2), (1024, 2080, 32, 1, 1), (16384, 4096, 64, 16, 0),
             (640, 544, 32, 3, 0), (512, 1024, 64, 40, 2)]
    problems = [(_problem(device, k, n, gs, m, 100 + i), k, n, gs, m, act) for i, (k, n, gs, m, act) in enumerate(calls)]
    want = [_with_workspace(hip, device, *p) for p in problems]
    assert want[0][1] > 0 and want[-1][1] == 0
    for _ in range(2):
        for p, (y_want, _) in zip(problems, want):
            assert_bits_equal(_no_alloc(hip, device, *p), y_want, str(p[1:]))


def test_no_alloc_entry_point_against_oracle(hip, device, oracle):
    """Not only equal to its sibling: the no-alloc entry point itself against the oracle's linear over
    the oracle-decompressed weight (the default layout of LinearGQ at a layer shape of the 6B stack),
    within the tolerance of the fused paths."""
    k_in, n_out, gs, m_rows = 4096, 4096, 64, 4
    tensors = _problem(device, k_in, n_out, gs, m_rows, 300)
    x, packed, scale, bias, out_bias = (t.cpu().numpy() for t in tensors)
    w = oracle.np_decompress(packed, scale, bias)  # [k_in, n_out]
    ref = oracle.np_linear(x, np.ascontiguousarray(w.T), out_bias)
    for _ in range(2):
        y = _no_alloc(hip, device, tensors, k_in, n_out, gs, m_rows, 0)
        err = np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max()
        assert err <= 1e-2, err


def test_no_alloc_entry_point_refuses_a_second_stream_while_the_first_is_busy(hip, device):
    """All calls on a GPU share the library's scratch array: a call on another stream while the first
    stream still has work pending is refused (nothing launched) instead of racing."""
    from popxl_addons._gq_hip import GQ_ERR_UNSUPPORTED, GQHipError

    k_in, n_out, gs, m_rows = 4096, 4096, 64, 2
    tensors = _problem(device, k_in, n_out, gs, m_rows, 301)
    x, packed, scale, bias, out_bias = tensors
    y = torch.empty((m_rows, n_out), dtype=torch.float16, device=device)

    def call(stream):
        hip.call("gq_linear_kn_act_noalloc_f16", x.data_ptr(), m_rows, packed.data_ptr(), scale.data_ptr(), bias.data_ptr(),
                 out_bias.data_ptr(), y.data_ptr(), n_out, k_in, gs, 0, stream.cuda_stream)

    other = torch.cuda.Stream(device=device)
    a = torch.randn((8192, 8192), dtype=torch.float16, device=device)
    torch.cuda.synchronize()
    for _ in range(40):  # tens of milliseconds of work on the current stream
        a @ a
    call(torch.cuda.current_stream())
    with pytest.raises(GQHipError) as refused:
        call(other)
    assert refused.value.code == GQ_ERR_UNSUPPORTED and "another stream" in str(refused.value)
    torch.cuda.synchronize()
    want = y.clone()
    y.fill_(float("nan"))
    torch.cuda.synchronize()  # (the copy and the fill are work of the first stream too)
    call(other)  # the first stream has drained
    torch.cuda.synchronize()
    assert torch.equal(want, y)


def test_no_alloc_entry_point_rejects_oversized_problems(hip, device):
    from popxl_addons._gq_hip import GQ_ERR_UNSUPPORTED, GQHipError

    n_out, gs, m_rows = 12288, 64, 16  # 48 strips x 6 K slabs x 8 batch-row pairs x 2 KiB = 4.5 MiB of partial sums
    need = hip.load().gq_linear_kn_workspace_bytes(m_rows, n_out, 4096, gs)
    assert need > (4 << 20) + 16384
    tensors = _problem(device, 64, 64, gs, m_rows, 1)  # (never launched: the sizes are rejected first)
    x, packed, scale, bias, out_bias = tensors
    with pytest.raises(GQHipError) as e:
        hip.call("gq_linear_kn_act_noalloc_f16", x.data_ptr(), m_rows, packed.data_ptr(), scale.data_ptr(), bias.data_ptr(),
                 0, x.data_ptr(), n_out, 4096, gs, 0, torch.cuda.current_stream().cuda_stream)
    assert e.value.code == GQ_ERR_UNSUPPORTED and "scratch" in str(e.value) and "workspace" in str(e.value)
