"""The device packer divides by the group's scale with ONE fp32 product per element: the difference
times the correctly rounded reciprocal of the scale (an IEEE division, once per group), rounded again
to fp16 (csrc/gq_compress.hip: divide).  This emulates that arithmetic with numpy for every pair of
11-bit significands over the binades a quotient can fall in, and checks that the result is the
correctly rounded fp16 quotient -- the value numpy computes in group_quantize_compress_numpy
(popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:192) -- wherever that
quotient is a normal fp16 number, and that the code made from it (:192, rint) is the same everywhere."""
import numpy as np
import pytest


def _code(q16):
    """1024 + q rounds to an integer, ties to even; the code is what is left of it, clipped at 15."""
    biased = np.minimum(q16 + np.float16(1024.0), np.float16(1039.0))
    return biased.view(np.uint16) & 0xF


@pytest.mark.parametrize("d_lo,d_hi", [(1, 1024), (1024, 2048)])
@pytest.mark.parametrize("power", [4, 3, 1, 0, -1, -5, -14, -20])
def test_product_with_rounded_reciprocal_is_correctly_rounded(d_lo, d_hi, power):
    d_sig = np.arange(d_lo, d_hi, dtype=np.float64) * 2.0**power
    s_sig = np.arange(1024, 2048, dtype=np.float64)
    d, s = np.meshgrid(d_sig, s_sig, indexing="ij")
    quotient = d / s
    want = quotient.astype(np.float16)  # 53 >= 2 * 11 + 2 bits: rounding the binary64 quotient again is exact
    r = (1.0 / s).astype(np.float32)  # correctly rounded (53 >= 2 * 24 + 2)
    product = d * r.astype(np.float64)  # 11 x 24 bits: exact in binary64
    got = product.astype(np.float32).astype(np.float16)
    normal = quotient >= 2.0**-14
    assert np.array_equal(got.view(np.uint16)[normal], want.view(np.uint16)[normal])
    assert np.array_equal(_code(got), _code(want))
    # the numpy packer's own rounding of the quotient
    in_range = want < np.float16(15.5)  # (beyond, the numpy packer's code does not fit four bits)
    assert np.array_equal(_code(want)[in_range], np.rint(want).astype(np.uint16)[in_range])


def test_distance_of_a_quotient_from_a_rounding_boundary():
    """The margin of the argument in the source: for 11-bit D, S a quotient in [1, 2) is at least
    1 / (S 2^11) away from every M / 2^11, M odd (a boundary of fp16 rounding)."""
    s = np.arange(1024, 2048, dtype=np.int64)[None, :]
    for shift in (11, 12):  # D >= S: D/S; D < S: 2D/S
        dd = np.arange(1024, 2048, dtype=np.int64)[:, None] << shift
        in_range = (dd >= (s << 11)) & (dd < (s << 12))
        # nearest odd M to dd / s: distance |dd - M s| / (s 2^11), numerator a non-zero integer
        m = (dd // s) | 1
        num = np.minimum(np.abs(dd - m * s), np.abs(dd - (m - 2) * s))
        num = np.minimum(num, np.abs(dd - (m + 2) * s))
        assert num[in_range].min() >= 1
