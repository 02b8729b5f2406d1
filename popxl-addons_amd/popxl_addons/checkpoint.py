"""On-disk format of quantised layers.

The layout is the reference's model-state convention (popxl_addons/task_session.py:203-214 for
writing, :239-266 for reading): a directory `<checkpoint_dir>/model/` holding one `.npz` file per
variable, the file named by the variable's dotted path (`layer.weight_compressed.npz`, ...) and
holding one array under that same name.  For a `LinearGQ` the variables are the three arrays of
the compressed weight and the optional additive bias (popxl_addons/layers/linear_gq.py:68,81,90,104).

`numpy.savez` stores its members uncompressed, so a variable can be memory-mapped straight out
of its `.npz` (`mmap=True`): a 6B-parameter stack then costs no host memory beyond the page cache
while it is copied to the GPU.  Files are read with `allow_pickle=False`.
"""
import glob
import logging
import os
import struct
import warnings
import zipfile
from typing import Dict, Mapping, Optional

import numpy as np

from popxl_addons.utils import _numpy_dtype_of

MODEL_DIR = "model"
REPORT_MISSING_METHODS = ("none", "warn", "error")


def _to_numpy(value):
    if isinstance(value, np.ndarray):
        return value
    if hasattr(value, "detach"):  # torch tensor
        import torch

        t = value.detach().cpu().contiguous()
        if t.dtype == torch.uint16:  # no direct numpy export for unsigned 16-bit tensors
            return t.view(torch.int16).numpy().view(np.uint16)
        return t.numpy()
    return np.asarray(value)


def variable_filename(checkpoint_dir: str, name: str) -> str:
    return os.path.join(checkpoint_dir, MODEL_DIR, f"{name}.npz")


def save_variables(checkpoint_dir: str, state: Mapping[str, object]) -> None:
    """Write every (dotted name -> array or tensor) of `state` as `<dir>/model/<name>.npz`."""
    os.makedirs(os.path.join(checkpoint_dir, MODEL_DIR), exist_ok=True)
    for name, value in state.items():
        np.savez(variable_filename(checkpoint_dir, name), **{name: _to_numpy(value)})


def _report_missing(found, expected, method):
    if method not in REPORT_MISSING_METHODS:
        raise ValueError(f"report_missing must be one of {REPORT_MISSING_METHODS}, got {method!r}")
    found, expected = set(found), set(expected)
    message = ""
    if expected - found:
        message += f"Missing keys: {sorted(expected - found)}. "
    if found - expected:
        message += f"Unexpected keys: {sorted(found - expected)}. "
    if message and method == "error":
        raise ValueError(message)
    if message and method == "warn":
        logging.warning(message)


def _mmap_member(filename: str, member: str) -> np.ndarray:
    """Memory-map the array stored (uncompressed) as `member` of the zip file `filename`."""
    with zipfile.ZipFile(filename) as zf:
        info = zf.getinfo(member)
        if info.compress_type != zipfile.ZIP_STORED:
            raise ValueError(f"{filename}: member {member} is compressed and cannot be memory-mapped")
        with open(filename, "rb") as f:
            # local file header: 30 fixed bytes, then the name and the extra field
            f.seek(info.header_offset)
            header = f.read(30)
            if header[:4] != b"PK\x03\x04":
                raise ValueError(f"{filename}: bad local header for {member}")
            name_len, extra_len = struct.unpack("<HH", header[26:30])
            data_start = info.header_offset + 30 + name_len + extra_len
            f.seek(data_start)
            version = np.lib.format.read_magic(f)
            if version == (1, 0):
                shape, fortran, dtype = np.lib.format.read_array_header_1_0(f)
            else:
                shape, fortran, dtype = np.lib.format.read_array_header_2_0(f)
            if dtype.hasobject:
                raise ValueError(f"{filename}: object arrays are not loaded")
            offset = f.tell()
    return np.memmap(filename, dtype=dtype, mode="r", offset=offset, shape=shape, order="F" if fortran else "C")


def load_variables(
    checkpoint_dir: str,
    expected: Optional[Mapping[str, object]] = None,
    report_missing: str = "warn",
    mmap: bool = False,
    prefix: str = "",
) -> Dict[str, np.ndarray]:
    """Read `<dir>/model/*.npz` into {dotted name: array}.

    expected  {name: variable} (anything with `.dtype` and `.shape`; torch or numpy dtypes) — only
              these names are loaded, differences between the two key sets are reported as
              `report_missing` says ("none", "warn", "error": task_session.py:24), and an array
              whose dtype or shape differs from its variable raises ValueError, as a WeightsDict
              does (popxl_addons/utils.py:79-99).  None: load every file.
    mmap      return read-only memory maps into the files instead of copies.
    prefix    look only at variables under this dotted path (one layer of a larger checkpoint).
    """
    files = {os.path.basename(f)[: -len(".npz")]: f for f in glob.glob(os.path.join(checkpoint_dir, MODEL_DIR, "*.npz"))}
    if prefix:
        files = {name: f for name, f in files.items() if name.startswith(prefix + ".")}
    if expected is not None:
        _report_missing(files.keys(), expected.keys(), report_missing)
        names = [n for n in expected if n in files]
    else:
        names = sorted(files)
    out = {}
    for name in names:
        if mmap:
            value = _mmap_member(files[name], f"{name}.npy")
        else:
            with np.load(files[name], allow_pickle=False) as loaded:
                value = loaded[name]
        if expected is not None:
            var = expected[name]
            want = var.dtype if isinstance(var.dtype, np.dtype) else _numpy_dtype_of(var.dtype)
            if np.dtype(want) != value.dtype:
                raise ValueError(f"{name}: variable and checkpoint dtypes do not equal {np.dtype(want)} != {value.dtype}")
            if tuple(var.shape) != tuple(value.shape):
                raise ValueError(f"{name}: variable and checkpoint shapes do not equal {tuple(var.shape)} != {tuple(value.shape)}")
        out[name] = value
    return out


def layer_state(prefix: str, variables) -> Dict[str, object]:
    """{dotted name: device tensor} of a layer's NamedTensors under `prefix` ("" for none)."""
    dot = f"{prefix}." if prefix else ""
    return {f"{dot}{name}": var.data for name, var in variables.items()}


def save_layer(checkpoint_dir: str, prefix: str, layer) -> None:
    """Write the variables of a built `LinearGQ` (or any object with `.variables`)."""
    if layer.variables is None:
        raise ValueError("save_layer: the layer has no variables yet (build it or call init_variables)")
    save_variables(checkpoint_dir, layer_state(prefix, layer.variables))


def load_layer(checkpoint_dir: str, prefix: str, layer, report_missing: str = "error", mmap: bool = True) -> None:
    """Copy `<dir>/model/<prefix>.<variable>.npz` into the layer's (already initialised) variables."""
    import torch

    if layer.variables is None:
        raise ValueError("load_layer: call init_variables(in_features, dtype, device) first")
    dot = f"{prefix}." if prefix else ""
    expected = {f"{dot}{name}": var for name, var in layer.variables.items()}
    arrays = load_variables(checkpoint_dir, expected, report_missing, mmap, prefix)
    for name, value in arrays.items():
        var = expected[name]
        host = np.ascontiguousarray(value)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)  # read-only memory map: it is only read
            if host.dtype == np.uint16:
                t = torch.from_numpy(host.view(np.int16)).view(torch.uint16)
            else:
                t = torch.from_numpy(host)
        var.data.copy_(t.to(var.data.device))
    if arrays and getattr(layer, "_decode_copy", None) is not None:
        layer.prepack_for_decode()  # (a derived copy of the variables: make it again)
