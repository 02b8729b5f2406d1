"""TEST INFRASTRUCTURE ONLY -- CPU oracle for the 4-bit group-quantization path.

Two independent restatements of the reference's algorithm live here:

* ``c_*``  : ctypes front end of ``gq_oracle.c`` (scalar C, every binary16 operation
  evaluated exactly and rounded once).  This is the bit-exactness checker.
* ``np_*`` : a numpy restatement that does the same array passes as
  ``popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:127-141``
  (decompress) and ``:172-196`` (compress).  It is what the benchmark times as the
  "reference numpy CPU path", and the tests hold it equal to the C oracle.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.

Pinning status (see tests/test_oracle_pinned.py):
  decompress   pinned (exact-rational brute force over all 65 536 words, seeded fixture of
               tests/integration/ops/test_group_quantize_decompress.py:15-42, invariants)
  compress     pinned (fixture relation packed==packed, scale within 1e-3, arg-min/arg-max
               codes, pack/unpack inverse, round-trip bound); constant groups (scale 0) are
               undefined in the reference and defined here as code 0
  linear       pinned (binary64 dot products vs numpy float32 matmul)
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgq_oracle.so")
_lib = None


def build(force=False):
    """Compile gq_oracle.c with gcc (make -C oracle)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        p, i64 = ctypes.c_void_p, ctypes.c_int64
        lib.gq_oracle_decompress.argtypes = [p, p, p, p, i64, i64, i64]
        lib.gq_oracle_decompress.restype = None
        for name in ("gq_oracle_compress_f16", "gq_oracle_compress_f32"):
            getattr(lib, name).argtypes = [p, p, p, p, i64, i64, i64]
            getattr(lib, name).restype = ctypes.c_int
        lib.gq_oracle_linear.argtypes = [p, p, p, p, i64, i64, i64]
        lib.gq_oracle_linear.restype = None
        lib.gq_oracle_f64_to_f16.argtypes = [ctypes.c_double]
        lib.gq_oracle_f64_to_f16.restype = ctypes.c_uint16
        lib.gq_oracle_f16_to_f64.argtypes = [ctypes.c_uint16]
        lib.gq_oracle_f16_to_f64.restype = ctypes.c_double
        _lib = lib
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _move_last_to(a, dim):
    # group_quantize_decompress.py:136-140: pop the last axis, list.insert it at `dim`
    if dim == -1:
        return a
    perm = list(range(a.ndim))
    last = perm.pop(-1)
    perm.insert(dim, last)
    return a.transpose(perm)


def _move_to_last(a, dim):
    # group_quantize_decompress.py:172-176: pop axis `dim`, append it
    if dim == -1:
        return a
    perm = list(range(a.ndim))
    perm.append(perm.pop(dim))
    return a.transpose(perm)


# --------------------------------------------------------------------------- C oracle


def c_f64_to_f16_bits(d):
    return int(_load().gq_oracle_f64_to_f16(float(d)))


def c_decompress(t, group_scale, group_bias, dim=-1):
    """Bit-exact oracle of group_quantize_decompress_numpy (…decompress.py:95-141)."""
    t = np.ascontiguousarray(t, dtype=np.uint16)
    lead, (g, i) = t.shape[:-2], t.shape[-2:]
    rows = int(np.prod(lead, dtype=np.int64)) if lead else 1
    s = np.ascontiguousarray(np.broadcast_to(np.asarray(group_scale, np.float16).reshape(*lead, g, 1), (*lead, g, 1)))
    b = np.ascontiguousarray(np.broadcast_to(np.asarray(group_bias, np.float16).reshape(*lead, g, 1), (*lead, g, 1)))
    out = np.empty((*lead, g * i * 4), dtype=np.float16)
    _load().gq_oracle_decompress(_ptr(t), _ptr(s), _ptr(b), _ptr(out), rows, g, i)
    return _move_last_to(out, dim)


def c_compress(t, group_size, dim=-1):
    """Oracle of group_quantize_compress_numpy (…decompress.py:144-196)."""
    t = np.ascontiguousarray(_move_to_last(np.asarray(t), dim))
    lead, n_cols = t.shape[:-1], t.shape[-1]
    g = n_cols // group_size
    rows = int(np.prod(lead, dtype=np.int64)) if lead else 1
    packed = np.empty((*lead, g, group_size // 4), dtype=np.uint16)
    scale = np.empty((*lead, g, 1), dtype=np.float16)
    bias = np.empty((*lead, g, 1), dtype=np.float16)
    if t.dtype == np.float16:
        fn = _load().gq_oracle_compress_f16
    elif t.dtype == np.float32:
        fn = _load().gq_oracle_compress_f32
    else:
        raise TypeError(f"oracle compress handles float16/float32 input, got {t.dtype}")
    rc = fn(_ptr(t), _ptr(packed), _ptr(scale), _ptr(bias), rows, g, group_size)
    if rc != 0:
        raise ValueError("Cannot compress t which contains non-finite values")
    return packed, scale, bias


def c_linear(x, w_dec, out_bias=None):
    """y = x @ w_dec.T (+ out_bias) with exact products, binary64 accumulation -> float32."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    w = np.ascontiguousarray(w_dec, dtype=np.float16)
    m, k = x.shape
    n = w.shape[0]
    assert w.shape[1] == k
    ob = None if out_bias is None else np.ascontiguousarray(out_bias, dtype=np.float16)
    y = np.empty((m, n), dtype=np.float32)
    _load().gq_oracle_linear(_ptr(x), _ptr(w), None if ob is None else _ptr(ob), _ptr(y), m, n, k)
    return y


# ----------------------------------------------------------------------- numpy oracle


def np_decompress(t, group_scale, group_bias, dim=-1):
    """Same array passes as group_quantize_decompress.py:127-141."""
    lead, (g, i) = t.shape[:-2], t.shape[-2:]
    nibbles = [(t >> shift) & 15 for shift in (12, 8, 4, 0)]  # :130, MSB nibble first
    codes = np.stack(nibbles, axis=-1).reshape(*lead, g, i * 4).astype(np.float16)  # :130-133
    vals = codes * group_scale  # binary16 multiply, rounded            (:134)
    vals = vals + group_bias  # then binary16 add, rounded: no fma      (:134)
    return _move_last_to(vals.reshape(*lead, g * i * 4), dim)  # :135-140


def np_compress(t, group_size, dim=-1):
    """Same array passes as group_quantize_decompress.py:172-196."""
    t = _move_to_last(t, dim)
    lead, n_cols = t.shape[:-1], t.shape[-1]
    if not np.isfinite(t).all():  # :182-183
        raise ValueError("Cannot compress t which contains non-finite values")
    grouped = t.reshape(*lead, n_cols // group_size, group_size)  # :185
    hi = grouped.max(-1, keepdims=True).astype(np.float16)  # :186
    lo = grouped.min(-1, keepdims=True).astype(np.float16)  # :187
    scale = (hi - lo) / 15  # :189 stays binary16
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.round((grouped - lo) / scale)  # :192 half-to-even
    q = np.where(scale == 0, 0, q).astype(np.uint16)  # constant group: undefined upstream
    weights = np.array([4096, 256, 16, 1], dtype=np.uint16)  # :193
    packed = (q.reshape(*lead, n_cols // group_size, group_size // 4, 4) * weights).sum(-1, dtype=np.uint16)  # :195
    return packed, scale, lo


def np_linear(x, w_dec, out_bias=None, activation=None):
    """fp32 matmul over the decompressed weight (tests/integration/layers/test_linear_gq.py:18-30,52),
    optionally followed by np_activation."""
    y = x.astype(np.float32) @ w_dec.astype(np.float32).T
    if out_bias is not None:
        y = y + out_bias.astype(np.float32)
    return np_activation(y, activation)


def np_activation(v, activation):
    """The epilogues of the fused entry points, in binary64.  No counterpart in the reference's
    path (its layer ends at the bias add, popxl_addons/layers/linear_gq.py:102-109): "relu" is
    max(v, 0); "gelu_tanh" is the tanh form of GELU, 0.5 v (1 + tanh(sqrt(2/pi) (v + 0.044715 v^3))).
    Pinned in tests/test_oracle_pinned.py by scalar evaluation with math.tanh and by identities."""
    if activation in (None, "none"):
        return v
    v64 = np.asarray(v, dtype=np.float64)
    if activation == "relu":
        return np.maximum(v64, 0.0)
    if activation == "gelu_tanh":
        return 0.5 * v64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v64 + 0.044715 * v64**3)))
    raise ValueError(f"unknown activation {activation!r}")
