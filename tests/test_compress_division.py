"""The device packer divides by the group's scale with a shared reciprocal and one Newton step
(csrc/gq_compress.hip: divide) instead of a full division per element.  This emulates that
arithmetic with numpy for every pair of 11-bit significands, with the hardware reciprocal off by
-1, 0 and +1 ulp, in three binades of the quotient (fp16-subnormal results included), and checks
that the result is the correctly rounded fp16 quotient -- the value numpy computes in
group_quantize_compress_numpy (popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:192)."""
import numpy as np
import pytest


def _shift_ulps(x, k):
    return (x.view(np.int32) + k).view(np.float32)


@pytest.mark.parametrize("d_lo,d_hi", [(1, 1024), (1024, 2048)])
@pytest.mark.parametrize("power", [0, 3, -5])
def test_shared_reciprocal_division_is_correctly_rounded(d_lo, d_hi, power):
    d_sig = np.arange(d_lo, d_hi, dtype=np.float64) * 2.0**power
    s_sig = np.arange(1024, 2048, dtype=np.float64)
    d, s = np.meshgrid(d_sig, s_sig, indexing="ij")
    want = (d / s).astype(np.float16)  # 53 >= 2 * 11 + 2 bits: rounding the binary64 quotient again is exact
    d32 = d.astype(np.float32)
    r0 = (1.0 / s).astype(np.float32)
    for k in (-1, 0, 1):
        r = _shift_ulps(r0.copy(), k)
        t = d32 * r
        residual = d - s * t.astype(np.float64)  # fma(-s, t, d)
        e = residual.astype(np.float32)
        assert np.array_equal(e.astype(np.float64), residual), "the residual must be exact in binary32"
        t2 = (t.astype(np.float64) + e.astype(np.float64) * r.astype(np.float64)).astype(np.float32)  # fma(e, r, t)
        got = t2.astype(np.float16)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (k, power)
