"""Writes the committed golden vectors of tests/golden/.  Run from the repo root:
    python tests/golden/make_golden.py

1. seeded_fixture_rows16.npz / seeded_fixture_checksums.json
   The seeded fixture recipe held by the reference's own test
   (tests/integration/ops/test_group_quantize_decompress.py:15-42): 4096 rows x 64 groups of 64,
   legacy np.random.seed(11235813), codes = randn.argsort(-1) % 16, limits from randn float16 with
   max + 0.1, and the expected tensor t built by that test's closed form
   t = float16(codes) * scale + bias.  The recipe is restated with plain numpy calls; no oracle or
   library code of this repository takes part, so the vectors are independent of what they check.
   The first 16 rows are stored whole; the full tensors are pinned by checksums.

2. edge_vectors.npz
   Hand-picked (scale, bias) pairs (subnormal, zero, negative, large, infinite) with the expected
   result of every code 0..15 computed by exact rational arithmetic (fractions.Fraction) and one
   explicit round-to-nearest-even to binary16 per operation.
"""
import hashlib
import json
import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def seeded_fixture():
    num_rows, num_groups, group_size = 4096, 64, 64
    np.random.seed(11235813)
    codes = (np.random.randn(num_rows, num_groups, group_size).argsort(-1) % 16).astype(np.uint16)
    nib = codes.reshape(num_rows, num_groups, group_size // 4, 4)
    packed = (nib[..., 0] * 4096 + nib[..., 1] * 256 + nib[..., 2] * 16 + nib[..., 3]).astype(np.uint16)
    lims = np.random.randn(num_rows, num_groups, 2).astype(np.float16)
    hi = lims.max(-1, keepdims=True) + 0.1
    lo = lims.min(-1, keepdims=True)
    scale = ((hi - lo) / 15).astype(np.float16)
    bias = lo.astype(np.float16)
    t = (codes.astype(np.float16) * scale + bias).reshape(num_rows, num_groups * group_size).astype(np.float16)
    return packed, scale, bias, t


# ---- exact binary16 arithmetic on rationals -------------------------------------------------


def f16_bits_to_fraction(bits):
    sign = -1 if bits >> 15 else 1
    e, m = (bits >> 10) & 31, bits & 1023
    if e == 31:
        return None  # inf / nan handled by the caller
    if e == 0:
        return sign * Fraction(m, 1 << 24)
    return sign * Fraction(m | 1024, 1) * Fraction(2) ** (e - 25)


def fraction_to_f16_bits(v, negative_zero=False):
    """Round-to-nearest-even to binary16; overflow gives infinity."""
    if v == 0:
        return 0x8000 if negative_zero else 0
    sign = 0x8000 if v < 0 else 0
    a = abs(v)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    q = max(e - 10, -24)
    n = a / Fraction(2) ** q
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    if lo >= 2048:
        lo //= 2
        q += 1
    if q > 5:
        return sign | 0x7C00
    if lo < 1024:
        return sign | lo
    return sign | ((q + 25) << 10) | (lo - 1024)


def exact_decompress_value(code, scale_bits, bias_bits):
    """binary16 bits of f16(f16(code * scale) + bias) with IEEE special-value rules."""
    s, b = f16_bits_to_fraction(scale_bits), f16_bits_to_fraction(bias_bits)
    s_nan = s is None and (scale_bits & 1023)
    b_nan = b is None and (bias_bits & 1023)
    if s_nan or b_nan:
        return 0x7E00
    if s is None:  # +-inf * code
        if code == 0:
            return 0x7E00
        prod_inf = 0x7C00 | (scale_bits & 0x8000)
        if b is None and (bias_bits & 0x8000) != (prod_inf & 0x8000):
            return 0x7E00
        return prod_inf
    prod_neg_zero = (code == 0 or s == 0) and bool(scale_bits & 0x8000)
    prod_bits = fraction_to_f16_bits(code * s, negative_zero=prod_neg_zero)
    if b is None:
        return bias_bits
    if (prod_bits & 0x7C00) == 0x7C00:
        return prod_bits
    p = f16_bits_to_fraction(prod_bits)
    total = p + b
    if total == 0:
        # x + (-x) = +0 ; (-0) + (-0) = -0 ; (+0) + (-0) = +0
        both_neg_zero = p == 0 and b == 0 and bool(prod_bits & 0x8000) and bool(bias_bits & 0x8000)
        return 0x8000 if both_neg_zero else 0
    return fraction_to_f16_bits(total)


EDGE_PAIRS = [
    # (scale bits, bias bits)
    (0x0000, 0x3C00),  # scale 0 -> bias
    (0x3C00, 0x0000),  # scale 1, bias 0 -> the code itself
    (0x0001, 0x0000),  # smallest subnormal scale
    (0x0001, 0x0001),
    (0x03FF, 0x8003),  # largest subnormal scale, negative subnormal bias
    (0x0400, 0x83FF),  # smallest normal scale
    (0x1C01, 0x9C03),  # ~0.004 scale typical of N(0, 0.02) weights
    (0x2003, 0xA7F1),
    (0x2E66, 0xB266),  # 0.1, -0.2
    (0x3555, 0xBBFF),  # 1/3, just under -1
    (0x6C00, 0xF000),  # 4096 * 15 = 61440 (finite), -8192
    (0x7000, 0x0000),  # 8192 * 8 overflows to inf for codes >= 8
    (0x7BFF, 0xFBFF),  # max * code overflows; + (-max)
    (0xB555, 0x3800),  # negative scale
    (0x8000, 0x8000),  # -0 * code + -0
    (0x7C00, 0x0000),  # inf scale: code 0 -> nan, others inf
    (0x3C00, 0x7C00),  # inf bias
    (0x7C00, 0xFC00),  # inf - inf -> nan
    (0x7E00, 0x3C00),  # nan scale
]


def main():
    packed, scale, bias, t = seeded_fixture()
    np.savez_compressed(
        os.path.join(HERE, "seeded_fixture_rows16.npz"),
        packed=packed[:16], scale=scale[:16], bias=bias[:16], t=t[:16],
    )
    sums = {
        "recipe": "tests/integration/ops/test_group_quantize_decompress.py:15-42, np.random.seed(11235813)",
        "packed_shape": list(packed.shape),
        "packed_sum": int(packed.astype(np.uint64).sum()),
        "packed_sha256": hashlib.sha256(packed.tobytes()).hexdigest(),
        "scale_sha256": hashlib.sha256(scale.tobytes()).hexdigest(),
        "bias_sha256": hashlib.sha256(bias.tobytes()).hexdigest(),
        "t_sha256": hashlib.sha256(t.tobytes()).hexdigest(),
        "t_row0_first4_bits": [int(v) for v in t[0, :4].view(np.uint16)],
    }
    with open(os.path.join(HERE, "seeded_fixture_checksums.json"), "w") as f:
        json.dump(sums, f, indent=1)

    rng = np.random.default_rng(20231)
    pairs = list(EDGE_PAIRS)
    # random finite pairs over the whole binary16 range (subnormals included)
    for _ in range(4096 - len(pairs)):
        s_bits = int(rng.integers(0, 0x7C00)) | (int(rng.integers(0, 2)) << 15)
        b_bits = int(rng.integers(0, 0x7C00)) | (int(rng.integers(0, 2)) << 15)
        pairs.append((s_bits, b_bits))
    scale_bits = np.array([p[0] for p in pairs], dtype=np.uint16)
    bias_bits = np.array([p[1] for p in pairs], dtype=np.uint16)
    expected = np.array(
        [[exact_decompress_value(c, int(s), int(b)) for c in range(16)] for s, b in zip(scale_bits, bias_bits)],
        dtype=np.uint16,
    )
    np.savez_compressed(
        os.path.join(HERE, "edge_vectors.npz"), scale_bits=scale_bits, bias_bits=bias_bits, expected_bits=expected
    )
    print(json.dumps(sums, indent=1))
    print("edge vectors:", expected.shape)


if __name__ == "__main__":
    main()
