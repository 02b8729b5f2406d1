"""4-bit group-quantized tensors: device decompress (HIP, gfx950) and the numpy compress /
decompress pair.

Same names, argument order and error behaviour as the reference module
popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py (`__all__` at :15-19);
the device op works on `torch.Tensor`s resident on the GPU instead of `popxl.Tensor`s.
`dim` defaults to -1 in the numpy pair as well, which is how the reference's own tests call
them (tests/integration/ops/test_group_quantize_decompress.py:47-48).

Scheme ("FlexGen", https://arxiv.org/abs/2303.06865): values are grouped along one axis; each
group keeps bias = min and scale = (max - min) / 15 in float16 and one 4-bit code per value;
four codes are packed into a uint16, most significant nibble first.
"""
from typing import Tuple

import numpy as np

from popxl_addons import _gq_hip

__all__ = [
    "group_quantize_decompress",
    "group_quantize_decompress_numpy",
    "group_quantize_compress_numpy",
    "group_quantize_compress",
]


def _perm_last_to(ndim: int, dim: int):
    # the reference's axis move (:87-91, :136-140): pop the last axis, list.insert it at `dim`
    perm = list(range(ndim))
    last = perm.pop(-1)
    perm.insert(dim, last)
    return perm


def _as_u16_ptr_tensor(t):
    import torch

    if t.dtype == torch.uint16:
        return t
    if t.dtype == torch.int16:
        return t.view(torch.uint16)
    raise TypeError(f"packed tensor must be uint16 (or an int16 view of it), got {t.dtype}")


def _stream_handle(device):
    import torch

    return torch.cuda.current_stream(device).cuda_stream


def group_quantize_decompress(t, group_scale, group_bias, dim=-1):
    """
    Decompress a 4-bit group-quantized tensor on the GPU.

    Args:
        t (torch.Tensor): packed codes, shape (num_rows, num_groups, num_group_ids), dtype uint16, on a HIP device
        group_scale (torch.Tensor): (num_rows, num_groups, 1) or (num_rows, num_groups), float16
        group_bias (torch.Tensor): same shape rules as group_scale, float16
        dim (int): where the decompressed axis is placed (list.insert semantics, -1 = last)

    Returns:
        torch.Tensor: float16, shape (num_rows, num_groups * num_group_ids * 4) with the last axis
        moved to `dim`; bit-identical to group_quantize_decompress_numpy.

    Checks mirror the reference wrapper (:57-73) and GroupQuantizeDecompressOp::setup
    (group_quantize_decompress.cpp:41-63).
    """
    import torch

    if t.dim() != 3:
        raise NotImplementedError("4-bit decompression currently supported only for packed tensors with rank 3")

    if group_scale.dim() < t.dim() - 1 or group_scale.dim() > t.dim():
        raise ValueError("group_scale.rank must be equal to or one less than t.rank")
    elif group_scale.dim() == t.dim() - 1:
        group_scale = group_scale.reshape(*group_scale.shape, 1)

    if group_bias.dim() < t.dim() - 1 or group_bias.dim() > t.dim():
        raise ValueError("group_bias.rank must be equal to or one less than t.rank")
    elif group_bias.dim() == t.dim() - 1:
        group_bias = group_bias.reshape(*group_bias.shape, 1)

    if tuple(t.shape[:-1]) != tuple(group_scale.shape[: t.dim() - 1]):
        raise ValueError("The first two dimensions of t and group_scale must be the same")
    if tuple(t.shape[:-1]) != tuple(group_bias.shape[: t.dim() - 1]):
        raise ValueError("The first two dimensions of t and group_bias must be the same")
    if group_scale.shape[2] != 1:
        raise ValueError("group_scale shape at last dimension should be 1")
    if group_bias.shape[2] != 1:
        raise ValueError("group_bias shape at last dimension should be 1")

    if not t.is_cuda:
        raise RuntimeError("group_quantize_decompress runs on the GPU only: move the tensors to a HIP device")
    if group_scale.device != t.device or group_bias.device != t.device:
        raise ValueError("t, group_scale and group_bias must be on the same device")
    if group_scale.dtype != torch.float16 or group_bias.dtype != torch.float16:
        raise TypeError("group_scale and group_bias must be float16")

    t = _as_u16_ptr_tensor(t).contiguous()
    group_scale = group_scale.contiguous()
    group_bias = group_bias.contiguous()
    rows, n_groups, n_ids = t.shape
    n_cols = n_groups * n_ids * 4

    transposed = dim != -1 and _perm_last_to(2, dim) != [0, 1]
    with torch.cuda.device(t.device):
        out = torch.empty((n_cols, rows) if transposed else (rows, n_cols), dtype=torch.float16, device=t.device)
        _gq_hip.call(
            "gq_decompress_f16_transposed" if transposed else "gq_decompress_f16",
            t.data_ptr(),
            group_scale.data_ptr(),
            group_bias.data_ptr(),
            out.data_ptr(),
            rows,
            n_groups,
            n_ids,
            _stream_handle(t.device),
        )
    return out


def group_quantize_compress(t, group_size: int, dim: int = -1):
    """
    Device-side compress of a float16 or float32 tensor (torch.Tensor on a HIP device): the same
    (packed, scale, bias) bits as group_quantize_compress_numpy gives for the same array (float32
    input is quantised in float32 arithmetic, as the reference does at :186-192).

    Raises ValueError for non-finite input, like the numpy function (:182-183).
    """
    import torch

    if not t.is_cuda:
        raise RuntimeError("group_quantize_compress runs on the GPU only")
    if t.dtype not in (torch.float16, torch.float32):
        raise TypeError("group_quantize_compress takes float16 or float32 input")
    if dim != -1:
        perm = list(range(t.dim()))
        perm.append(perm.pop(dim))
        t = t.permute(perm)
    t = t.contiguous()
    lead, n_cols = tuple(t.shape[:-1]), t.shape[-1]
    if group_size <= 0 or group_size % 4 != 0 or n_cols % group_size != 0:
        raise ValueError(f"group_size={group_size} must be a multiple of 4 that divides {n_cols}")
    n_groups = n_cols // group_size
    rows = 1
    for d in lead:
        rows *= d
    with torch.cuda.device(t.device):
        packed = torch.empty((*lead, n_groups, group_size // 4), dtype=torch.uint16, device=t.device)
        scale = torch.empty((*lead, n_groups, 1), dtype=torch.float16, device=t.device)
        bias = torch.empty((*lead, n_groups, 1), dtype=torch.float16, device=t.device)
        flag = torch.zeros(1, dtype=torch.int32, device=t.device)
        _gq_hip.call(
            "gq_compress_f16" if t.dtype == torch.float16 else "gq_compress_f32",
            t.data_ptr(),
            packed.data_ptr(),
            scale.data_ptr(),
            bias.data_ptr(),
            flag.data_ptr(),
            rows,
            n_groups,
            group_size,
            _stream_handle(t.device),
        )
        if int(flag.item()) != 0:
            raise ValueError("Cannot compress t which contains non-finite values")
    return packed, scale, bias


def group_quantize_decompress_numpy(
    t: np.ndarray, group_scale: np.ndarray, group_bias: np.ndarray, dim: int = -1
) -> np.ndarray:
    """
    Numpy decompress (host).  value = float16(float16(code * scale) + bias).

    Args:
        t: packed codes, shape (*leading, num_groups, num_group_ids), uint16
        group_scale, group_bias: shape (*leading, num_groups, 1), float16
        dim: where the decompressed axis goes (-1 keeps it last)

    Returns:
        float16 array of shape (*leading, num_groups * num_group_ids * 4), last axis moved to `dim`.
    """
    t = np.asarray(t)
    lead, (n_groups, n_ids) = t.shape[:-2], t.shape[-2:]
    vals = np.empty((*lead, n_groups, n_ids, 4), dtype=np.float16)
    for j in range(4):  # nibble j of every word, most significant first
        vals[..., j] = (t >> (12 - 4 * j)) & 15
    vals = vals.reshape(*lead, n_groups, n_ids * 4)
    vals = np.multiply(vals, np.asarray(group_scale, dtype=np.float16), out=vals)  # rounded to float16
    vals = np.add(vals, np.asarray(group_bias, dtype=np.float16), out=vals)  # rounded again: not an fma
    vals = vals.reshape(*lead, n_groups * n_ids * 4)
    if dim != -1:
        vals = vals.transpose(_perm_last_to(vals.ndim, dim))
    return vals


def group_quantize_compress_numpy(
    t: np.ndarray, group_size: int, dim: int = -1
) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """
    Numpy compress (host).

    Args:
        t: float16 or float32 array; axis `dim` is grouped and must be a multiple of group_size
        group_size: values per (scale, bias) pair, a multiple of 4
        dim: axis to quantize along

    Returns:
        packed uint16 (*other_dims, num_groups, group_size // 4),
        scale float16 (*other_dims, num_groups, 1), bias float16 (*other_dims, num_groups, 1)

    Arithmetic follows the reference (:186-192): max/min are cast to float16 first, the scale is
    float16, and (x - bias) / scale is evaluated in t's own precision with round-half-to-even.
    Two cases the reference leaves undefined are defined here: a constant group (scale 0) gets
    code 0 everywhere, and codes are clipped to [0, 15].
    """
    t = np.asarray(t)
    if dim != -1:
        perm = list(range(t.ndim))
        perm.append(perm.pop(dim))
        t = t.transpose(perm)
    lead, n_cols = t.shape[:-1], t.shape[-1]
    if group_size <= 0 or group_size % 4 != 0 or n_cols % group_size != 0:
        raise ValueError(f"group_size={group_size} must be a multiple of 4 that divides {n_cols}")
    if not np.isfinite(t).all():
        raise ValueError("Cannot compress t which contains non-finite values")

    n_groups = n_cols // group_size
    grouped = t.reshape(*lead, n_groups, group_size)
    hi = grouped.max(axis=-1, keepdims=True).astype(np.float16)
    lo = grouped.min(axis=-1, keepdims=True).astype(np.float16)
    scale = (hi - lo) / np.float16(15)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint((grouped - lo) / scale)
    q = np.where(scale == 0, 0, q)
    q = np.clip(q, 0, 15).astype(np.uint16).reshape(*lead, n_groups, group_size // 4, 4)
    packed = (q[..., 0] << 12) | (q[..., 1] << 8) | (q[..., 2] << 4) | q[..., 3]
    return packed.astype(np.uint16), scale, lo
