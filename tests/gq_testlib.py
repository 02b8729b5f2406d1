"""Shared helpers of the GPU parity tests: seeded workloads of the benchmark configurations and the
comparison rules (bit-exact for decompress/compress, max-abs-normalised 1e-2 for the fused paths)."""
import numpy as np


def config2_weight(rows=4096, cols=16384, seed=2):
    """~N(0, 0.02) weight with 0.1 % outliers at +-8 sigma (benchmark configuration 2)."""
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    mask = rng.random((rows, cols)) < 1e-3
    sign = np.where(rng.random((rows, cols)) < 0.5, -1.0, 1.0)
    w[mask] = (0.16 * sign[mask]).astype(np.float32)
    return w.astype(np.float16)


def normal_weight(n_out, k_in, seed):
    return np.random.default_rng(seed).normal(0, 0.02, (n_out, k_in)).astype(np.float16)


def activations(m_rows, k_in, seed):
    return np.random.default_rng(seed).normal(0, 1, (m_rows, k_in)).astype(np.float16)


def is_nan16(bits):
    return ((bits & 0x7C00) == 0x7C00) & ((bits & 0x3FF) != 0)


def assert_bits_equal(got, want, what=""):
    """fp16 arrays equal bit for bit; NaNs need only be NaNs (payload/sign are not part of the contract)."""
    g, w = np.ascontiguousarray(got).view(np.uint16), np.ascontiguousarray(want).view(np.uint16)
    assert g.shape == w.shape, f"{what}: shape {g.shape} != {w.shape}"
    ng, nw = is_nan16(g), is_nan16(w)
    assert np.array_equal(ng, nw), f"{what}: NaN positions differ"
    bad = (g != w) & ~ng
    assert not bad.any(), f"{what}: {int(bad.sum())} of {g.size} values differ, first at {np.argwhere(bad)[0]}"


def normalised_error(y_gpu, y_ref):
    y_ref = np.asarray(y_ref, dtype=np.float64)
    return float(np.abs(np.asarray(y_gpu, dtype=np.float64) - y_ref).max() / max(np.abs(y_ref).max(), 1e-30))


def to_dev(a, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(device)
