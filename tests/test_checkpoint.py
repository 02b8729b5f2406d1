"""On-disk format of quantised layers: one .npz per variable under <dir>/model/, named by dotted
path, one array of the same name inside (the layout written by the reference's
popxl_addons/task_session.py:203-214 and read back at :239-266)."""
import logging
import os

import numpy as np
import pytest

from popxl_addons import checkpoint
from popxl_addons.layers.linear_gq import LinearGQ
from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy


class Var:
    def __init__(self, array):
        self.dtype, self.shape = array.dtype, array.shape


def _state(seed=3, out_features=32, in_features=128, group_size=16):
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (out_features, in_features)).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, group_size)
    return {
        "layers.0.attention.qkv.weight_compressed": packed,
        "layers.0.attention.qkv.weight_decompression_scale": scale,
        "layers.0.attention.qkv.weight_decompression_bias": bias,
        "layers.0.attention.qkv.bias": rng.normal(0, 1, (out_features,)).astype(np.float16),
    }


def test_layout_is_one_npz_per_variable(tmp_path):
    state = _state()
    checkpoint.save_variables(str(tmp_path), state)
    files = sorted(os.listdir(tmp_path / "model"))
    assert files == sorted(f"{name}.npz" for name in state)
    # what the reference's loader does with such a file (task_session.py:255-258)
    for name, value in state.items():
        with np.load(tmp_path / "model" / f"{name}.npz", allow_pickle=False) as loaded:
            assert loaded.files == [name]
            assert loaded[name].dtype == value.dtype
            np.testing.assert_array_equal(loaded[name], value)


@pytest.mark.parametrize("mmap", [False, True])
def test_round_trip(tmp_path, mmap):
    state = _state()
    checkpoint.save_variables(str(tmp_path), state)
    expected = {name: Var(value) for name, value in state.items()}
    loaded = checkpoint.load_variables(str(tmp_path), expected, report_missing="error", mmap=mmap)
    assert set(loaded) == set(state)
    for name, value in state.items():
        assert loaded[name].dtype == value.dtype and loaded[name].shape == value.shape
        np.testing.assert_array_equal(np.asarray(loaded[name]), value)
        assert isinstance(loaded[name], np.memmap) == mmap


def test_missing_and_unexpected_keys(tmp_path, caplog):
    state = _state()
    checkpoint.save_variables(str(tmp_path), state)
    expected = {name: Var(value) for name, value in state.items()}
    expected["layers.0.attention.out.weight_compressed"] = Var(np.zeros((2, 2, 2), np.uint16))
    del expected["layers.0.attention.qkv.bias"]
    with pytest.raises(ValueError, match="Missing keys.*out.weight_compressed.*Unexpected keys.*qkv.bias"):
        checkpoint.load_variables(str(tmp_path), expected, report_missing="error")
    with caplog.at_level(logging.WARNING):
        loaded = checkpoint.load_variables(str(tmp_path), expected, report_missing="warn")
    assert "Missing keys" in caplog.text
    assert set(loaded) == set(expected) - {"layers.0.attention.out.weight_compressed"}
    caplog.clear()
    with caplog.at_level(logging.WARNING):
        checkpoint.load_variables(str(tmp_path), expected, report_missing="none")
    assert caplog.text == ""
    with pytest.raises(ValueError):
        checkpoint.load_variables(str(tmp_path), expected, report_missing="loudly")


def test_dtype_and_shape_are_checked(tmp_path):
    state = _state()
    checkpoint.save_variables(str(tmp_path), state)
    name = "layers.0.attention.qkv.weight_compressed"
    with pytest.raises(ValueError, match="dtypes do not equal"):
        checkpoint.load_variables(str(tmp_path), {name: Var(state[name].astype(np.int32))}, report_missing="none")
    with pytest.raises(ValueError, match="shapes do not equal"):
        checkpoint.load_variables(str(tmp_path), {name: Var(state[name][:, :, :2])}, report_missing="none")


def test_pickled_members_are_refused(tmp_path):
    os.makedirs(tmp_path / "model")
    np.savez(tmp_path / "model" / "v.npz", v=np.array([{"a": 1}], dtype=object))
    with pytest.raises(ValueError):
        checkpoint.load_variables(str(tmp_path), None)
    with pytest.raises(ValueError):
        checkpoint.load_variables(str(tmp_path), None, mmap=True)


def test_layer_round_trip_on_host_tensors(tmp_path):
    import torch

    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.02, (128, 256)).astype(np.float16)  # [in, out]
    layer = LinearGQ(256, bias=True, group_size=16, dim=0)
    variables = layer.init_variables(128, torch.float16, torch.device("cpu"))
    packed, scale, bias = group_quantize_compress_numpy(w.T.copy(), 16)
    layer.load_weights({variables.weight_compressed: packed, variables.weight_decompression_scale: scale,
                        variables.weight_decompression_bias: bias,
                        variables.bias: rng.normal(0, 1, (256,)).astype(np.float16)})
    checkpoint.save_layer(str(tmp_path), "decoder.ff1", layer)
    checkpoint.save_variables(str(tmp_path), {"decoder.ff2.bias": np.zeros(4, np.float16)})  # another layer's file
    assert sorted(f for f in os.listdir(tmp_path / "model") if f.startswith("decoder.ff1.")) == sorted(
        f"decoder.ff1.{n}.npz" for n in ("weight_compressed", "weight_decompression_scale", "weight_decompression_bias", "bias"))

    other = LinearGQ(256, bias=True, group_size=16, dim=0)
    other.init_variables(128, torch.float16, torch.device("cpu"))
    checkpoint.load_layer(str(tmp_path), "decoder.ff1", other)
    for name, var in layer.variables.items():
        assert torch.equal(var.data.view(torch.int16), other.variables[name].data.view(torch.int16)), name

    no_bias = LinearGQ(256, bias=False, group_size=16, dim=0)
    no_bias.init_variables(128, torch.float16, torch.device("cpu"))
    with pytest.raises(ValueError, match="Unexpected keys"):
        checkpoint.load_layer(str(tmp_path), "decoder.ff1", no_bias)
    checkpoint.load_layer(str(tmp_path), "decoder.ff1", no_bias, report_missing="none")
