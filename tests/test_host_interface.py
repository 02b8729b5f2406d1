"""Host-side logic that needs no GPU: the C-ABI library loads and exports what the header
declares, the op wrapper and the layer validate their arguments like the reference."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT
from popxl_addons import _gq_hip
from popxl_addons.layers.linear_gq import LinearGQ
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy, group_quantize_decompress
from popxl_addons.utils import NamedTensors, Variable, WeightsDict


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "gq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 9
    assert sorted(names) == sorted(_gq_hip.EXPORTS)
    lib = ctypes.CDLL(_gq_hip.library_path())
    for n in names:
        assert getattr(lib, n) is not None


def test_every_entry_point_has_its_reference_interface_written_down():
    """The integration notes name, for every declared entry point, the reference interface it stands
    for (or say that it has none), and name no entry point that does not exist."""
    with open(os.path.join(ROOT, "INTEGRATION.md")) as f:
        table = [line for line in f if line.startswith("| `gq_")]
    listed = set(re.findall(r"`(gq_[a-z0-9_]+)`", " ".join(line.split("|")[1] for line in table)))
    assert listed == set(_declared_functions())


def test_abi_version_and_error_text_without_gpu():
    lib = _gq_hip.load()
    assert lib.gq_abi_version() == _gq_hip.GQ_ABI_VERSION
    # argument errors are detected before any device call
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_decompress_f16", 0, 0, 0, 0, 4, 4, 4, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER and "NULL" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_decompress_f16", 16, 16, 16, 16, -1, 4, 4, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_decompress_f16", 17, 16, 16, 16, 1, 4, 4, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_f16", 16, 1, 16, 16, 16, 0, 16, 8, 96, 64, None)  # 96 % 64 != 0
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_f16", 16, 17, 16, 16, 16, 0, 16, 8, 64, 64, None)  # m_rows > 16
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_f16", 16, 1, 16, 16, 16, 0, 16, 8, 64, 6, None)  # group_size % 4
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    # the layer's entry with the weight's streaming-layout copy: the copy alone (packed, scale, bias NULL) takes an aligned x
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_act_f16", 18, 1, 0, 0, 0, 16, 0, 16, 8, 512, 64, 0, None, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED and "16-byte" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_act_f16", 16, 1, 0, 16, 16, 16, 0, 16, 8, 512, 64, 0, None, 0, None)  # packed NULL, scale and bias not
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_act_f16", 16, 1, 16, 16, 16, 16, 0, 16, 8, 448, 64, 0, None, 0, None)  # no copy exists for k_in = 448
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "512" in str(e.value)
    # the same entry for an x whose rows are a stride apart: decode batches only, a stride of at least k_in, and with the
    # copy alone every row of x on a 16-byte boundary
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_strided_f16", 16, 1024, 17, 16, 16, 16, 16, 0, 16, 8, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "16 rows" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_strided_f16", 16, 500, 4, 16, 16, 16, 16, 0, 16, 8, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE and "x_row_stride" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_strided_f16", 16, 1028, 4, 0, 0, 0, 16, 0, 16, 8, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED and "x_row_stride" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_p_strided_f16", 16, 1024, 4, 16, 0, 16, 16, 0, 16, 8, 512, 64, 0, None)  # scale NULL, the others not
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_knp_strided_f16", 16, 1024, 17, 16, 0, 16, 64, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "16 rows" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_knp_strided_f16", 16, 1028, 4, 16, 0, 16, 64, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED and "x_row_stride" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_knp_strided_f16", 16, 256, 4, 16, 0, 16, 64, 512, 64, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    # the [k_in, n_out] layout: its own argument rules and the workspace contract
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_kn_act_f16", 16, 1, 16, 16, 16, 0, 16, 96, 64, 64, 0, None, 0, None)  # 96 % 64 != 0
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE and "n_out" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_kn_act_f16", 16, 1, 16, 16, 16, 0, 16, 128, 64, 64, 3, None, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "activation" in str(e.value)
    need = lib.gq_linear_kn_workspace_bytes(1, 16384, 4096, 64)
    assert need > 16384 and need <= 16384 + 64 * 16384 * 4 and need == lib.gq_linear_kn_workspace_bytes(1, 16384, 4096, 32)
    assert lib.gq_linear_kn_workspace_bytes(4, 16384, 4096, 64) == 16384 + (need - 16384) * 2  # two batch-row pairs
    assert lib.gq_linear_kn_workspace_bytes(1, 128, 64, 64) == 0  # one K slab: no scratch
    assert lib.gq_linear_kn_workspace_bytes(300, 16384, 4096, 64) == 0  # prefill batches with tiles enough for the device need none
    # ... with few tiles the prefill kernel divides K over workgroups: counters + 64 KiB per (slab, tile)
    assert lib.gq_linear_kn_workspace_bytes(128, 16384, 4096, 64) == 16384 + 2 * 128 * 65536
    assert lib.gq_linear_kn_workspace_bytes(300, 4096, 16384, 64) == 16384 + 3 * 96 * 65536
    assert lib.gq_linear_kn_workspace_bytes(17, 16384, 4096, 64) == 16384 + 2 * 128 * 65536
    assert lib.gq_linear_kn_workspace_bytes(1, 16384, 4096, 20) == 0  # generic kernel
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_kn_act_f16", 16, 1, 16, 16, 16, 0, 16, 16384, 4096, 64, 0, None, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER and "workspace" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_kn_act_f16", 16, 1, 16, 16, 16, 0, 16, 16384, 4096, 64, 0, 256, need - 1, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE and "workspace" in str(e.value)
    # the sequence with a caller-owned workspace
    assert lib.gq_gemv_sequence_workspace_bytes() == (256 + 4 + 4) * 128 + (32 << 20)  # progress lines, 3 + 4 words, two 16 MiB exchanges
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_ws_f16", 16, 16, 1, None, None, 0, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER and "workspace" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_ws_f16", 16, 16, 1, None, 256, 100, 0, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    # device packer for binary32 input
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_compress_f32", 16, 16, 16, 16, 0, 4, 4, 6, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_compress_f32", 18, 16, 16, 16, 0, 4, 4, 8, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED
    # sequence descriptors are validated on the host copy: an entry cannot wait for itself
    import numpy as np

    desc = np.zeros(2, dtype=np.dtype([("ptrs", "<u8", 6), ("ints", "<i4", 6)]))
    assert desc.dtype.itemsize == 72
    desc["ptrs"] = [[16, 16, 16, 16, 0, 16]] * 2
    desc["ints"] = [[1, 8, 64, 64, 0, 0], [1, 8, 64, 64, 2, 0]]  # m_rows n_out k_in group_size wait_entries reserved
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", desc.ctypes.data, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_BAD_SHAPE and "wait_entries" in str(e.value)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", 0, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER
    _gq_hip.call("gq_gemv_sequence_f16", 0, 0, 0, None, None)  # empty sequence
    # an unknown activation is rejected before anything is launched
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_linear_act_f16", 16, 1, 16, 16, 16, 0, 16, 8, 64, 64, 7, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "activation" in str(e.value)
    desc["ints"] = [[1, 8, 64, 64, 0, 0], [1, 8, 64, 64, 1, 9]]
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", desc.ctypes.data, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "activation" in str(e.value)
    # the streaming layout: its size, what it needs, and what an entry that uses it needs
    lib = _gq_hip.load()
    assert lib.gq_gemv_prepacked_bytes(4096, 4096, 64) == 256 * 8 * 4608 == int(4096 * 4096 * 0.5625)
    assert lib.gq_gemv_prepacked_bytes(1000, 1536, 64) == 63 * 3 * 4608  # rows padded to 16
    assert lib.gq_gemv_prepacked_bytes(0, 512, 64) == 0
    assert lib.gq_gemv_prepacked_bytes(64, 512, 32) == _gq_hip.GQ_ERR_UNSUPPORTED
    assert lib.gq_gemv_prepacked_bytes(64, 448, 64) == _gq_hip.GQ_ERR_UNSUPPORTED and "512" in _gq_hip.last_error()
    assert lib.gq_gemv_prepacked_bytes(-1, 512, 64) == _gq_hip.GQ_ERR_BAD_SHAPE
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_prepack_f16", 16, 16, 16, 0, 64, 512, 64, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_prepack_f16", 16, 16, 8, 16, 64, 512, 64, None)
    assert e.value.code == _gq_hip.GQ_ERR_MISALIGNED
    desc["ptrs"] = [[16, 16, 16, 16, 0, 16], [16, 16, 0, 0, 0, 16]]  # entry 1: scale == bias == NULL
    desc["ints"] = [[1, 8, 512, 64, 0, 0], [17, 8, 512, 64, 1, 0]]  # (more than 16 rows)
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", desc.ctypes.data, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "streaming layout" in str(e.value)
    desc["ints"] = [[1, 8, 512, 64, 0, 0], [1, 8, 512, 32, 1, 0]]
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", desc.ctypes.data, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_UNSUPPORTED and "streaming layout" in str(e.value)
    desc["ptrs"] = [[16, 16, 16, 16, 0, 16], [16, 16, 0, 16, 0, 16]]  # only scale NULL: not a blob, an error
    desc["ints"] = [[1, 8, 512, 64, 0, 0], [1, 8, 512, 64, 1, 0]]
    with pytest.raises(_gq_hip.GQHipError) as e:
        _gq_hip.call("gq_gemv_sequence_f16", desc.ctypes.data, 16, 2, None, None)
    assert e.value.code == _gq_hip.GQ_ERR_NULL_POINTER
    assert _gq_hip.activation_code("gelu_tanh") == _gq_hip.GQ_ACT_GELU_TANH and _gq_hip.activation_code(None) == 0
    with pytest.raises(ValueError):
        _gq_hip.activation_code("swish")
    # zero-sized problems succeed without touching a device
    _gq_hip.call("gq_decompress_f16", 0, 0, 0, 0, 0, 4, 4, None)
    _gq_hip.call("gq_gemv_f16", 0, 0, 0, 0, 0, 0, 0, 8, 64, 64, None)
    _gq_hip.call("gq_compress_f16", 0, 0, 0, 0, 0, 0, 4, 64, None)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setenv("GQ_HIP_LIBRARY", "/nonexistent/libgq_hip.so")
    monkeypatch.setattr(_gq_hip, "_lib", None)
    with pytest.raises(ImportError):
        _gq_hip.load()


def test_op_argument_validation():
    """Exceptions of the reference wrapper (group_quantize_decompress.py:57-73) and of
    GroupQuantizeDecompressOp::setup (group_quantize_decompress.cpp:41-63)."""
    t = torch.zeros((4, 2, 3), dtype=torch.uint16)
    s = torch.zeros((4, 2, 1), dtype=torch.float16)
    with pytest.raises(NotImplementedError):
        group_quantize_decompress(torch.zeros((4, 6), dtype=torch.uint16), s, s)
    with pytest.raises(NotImplementedError):
        group_quantize_decompress(torch.zeros((1, 4, 2, 3), dtype=torch.uint16), s, s)
    with pytest.raises(ValueError, match="group_scale.rank"):
        group_quantize_decompress(t, torch.zeros((4,), dtype=torch.float16), s)
    with pytest.raises(ValueError, match="group_bias.rank"):
        group_quantize_decompress(t, s, torch.zeros((4, 2, 1, 1), dtype=torch.float16))
    with pytest.raises(ValueError, match="t and group_scale"):
        group_quantize_decompress(t, torch.zeros((4, 3, 1), dtype=torch.float16), s)
    with pytest.raises(ValueError, match="t and group_bias"):
        group_quantize_decompress(t, s, torch.zeros((5, 2), dtype=torch.float16))
    with pytest.raises(ValueError, match="last dimension"):
        group_quantize_decompress(t, torch.zeros((4, 2, 2), dtype=torch.float16), s)
    # rank-2 scale/bias are accepted (reshaped to (..., 1)); a CPU tensor is then refused: no fallback
    with pytest.raises(RuntimeError, match="GPU only"):
        group_quantize_decompress(t, torch.zeros((4, 2), dtype=torch.float16), s)


def test_linear_gq_variables_and_mapping():
    """Variable names, shapes and dtypes of LinearGQ.build (linear_gq.py:67-108) and torch_mapping (:112-136)."""
    torch.manual_seed(0)
    nn_layer = torch.nn.Linear(128, 256, bias=True)
    for dim, packed_shape in ((0, (256, 8, 4)), (-1, (128, 16, 4)), (1, (128, 16, 4))):
        layer = LinearGQ(256, bias=True, group_size=16, dim=dim)
        v = layer.init_variables(128, torch.float16, "cpu")
        assert list(v.keys()) == ["weight_compressed", "weight_decompression_scale", "weight_decompression_bias", "bias"]
        assert v.weight_compressed.shape == packed_shape and v.weight_compressed.dtype == torch.uint16
        assert v.weight_decompression_scale.shape == (*packed_shape[:2], 1)
        assert v.weight_decompression_bias.dtype == torch.float16 and v.bias.shape == (256,)
        w = LinearGQ.torch_mapping(v, nn_layer, dtype=torch.float16, group_size=16, dim=dim)
        assert len(w) == 4
        want = group_quantize_compress_numpy(nn_layer.weight.T.detach().numpy(), 16, dim=dim)
        assert np.array_equal(w[v.weight_compressed], want[0])
        layer.load_weights(w)
        assert np.array_equal(v.weight_compressed.data.numpy(), want[0])
    assert "bias" not in LinearGQ(8, bias=False, group_size=4).init_variables(8, torch.float16, "cpu")


@pytest.mark.parametrize("dim", [0, -1])
def test_linear_gq_fused_variables(oracle, dim):
    """LinearGQ.fuse (outputs side by side) and LinearGQ.fuse_inputs (inputs side by side, results
    added): the stacked variables decompress to the layers' [in, out] weights laid side by side."""
    torch.manual_seed(1)

    def layer_of(n_in, n_out):
        nn_layer = torch.nn.Linear(n_in, n_out, bias=True)
        layer = LinearGQ(n_out, bias=True, group_size=16, dim=dim)
        v = layer.init_variables(n_in, torch.float16, "cpu")
        layer.load_weights(LinearGQ.torch_mapping(v, nn_layer, dtype=torch.float16, group_size=16, dim=dim))
        return layer

    def weight_in_out(layer):
        v = layer.variables
        w = oracle.np_decompress(*(v[n].data.numpy() for n in ("weight_compressed", "weight_decompression_scale", "weight_decompression_bias")))
        return w.T if dim == 0 else w  # dim=0 keeps [out, in]

    a, b = layer_of(64, 48), layer_of(64, 80)
    wide = LinearGQ.fuse([a, b])
    assert wide.out_features == 128
    assert np.array_equal(weight_in_out(wide), np.concatenate([weight_in_out(a), weight_in_out(b)], axis=1))
    assert np.array_equal(wide.variables.bias.data.numpy(), np.concatenate([a.variables.bias.data.numpy(), b.variables.bias.data.numpy()]))
    c, d = layer_of(64, 48), layer_of(96, 48)
    deep = LinearGQ.fuse_inputs([c, d])
    assert deep.out_features == 48
    assert np.array_equal(weight_in_out(deep), np.concatenate([weight_in_out(c), weight_in_out(d)], axis=0))
    total = (c.variables.bias.data.float() + d.variables.bias.data.float()).to(torch.float16)
    assert np.array_equal(deep.variables.bias.data.numpy(), total.numpy())
    with pytest.raises(ValueError):
        LinearGQ.fuse_inputs([a, b])  # other output widths
    with pytest.raises(ValueError):
        LinearGQ.fuse_inputs([])


def test_linear_gq_misuse():
    with pytest.raises(ZeroDivisionError):  # group_size left at its default 0 (linear_gq.py:25,73)
        LinearGQ(8).init_variables(8, torch.float16, "cpu")
    with pytest.raises(NotImplementedError):
        LinearGQ(8, replica_grouping=object(), group_size=4)
    with pytest.raises(ValueError):
        LinearGQ(8, group_size=4, dim=2).init_variables(8, torch.float16, "cpu")
    with pytest.raises(RuntimeError, match="GPU only"):
        LinearGQ(8, group_size=4, dim=0).build(torch.zeros((1, 8), dtype=torch.float16))


def test_weights_dict_validates_dtype_and_shape():
    """popxl_addons/utils.py:91-99."""
    var = Variable("w", torch.zeros((2, 3), dtype=torch.float16))
    d = WeightsDict()
    d[var] = np.zeros((2, 3), np.float16)
    with pytest.raises(ValueError, match="dtypes"):
        d[var] = np.zeros((2, 3), np.float32)
    with pytest.raises(ValueError, match="shapes"):
        d[var] = np.zeros((3, 2), np.float16)
    nt = NamedTensors(w=var)
    assert nt.w is var and nt["w"] is var and "w" in nt
    with pytest.raises(AttributeError):
        nt.missing
