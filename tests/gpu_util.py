"""Helpers shared by the GPU parity tests (they all go through the C ABI)."""
import numpy as np
import torch

from oracle import cpu
from tests.util import lut_bytes, lut_path


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def lut32(kind, m):
    return cpu.expand_u8(lut_bytes(kind, m), m)


def asym_lut_u8(m=3):
    """Asymmetric table (entry depends on operand order), as LUT-file bytes."""
    n = 1 << m
    i, j = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32), indexing="ij")
    return ((((i > j).astype(np.uint32)) << 7) | ((i * 3 + j * 5 + 1) % n)).astype(np.uint8).ravel()


def assert_close_sum_abs(got, want, sum_abs, rel=1e-5):
    """|got - want| <= rel * sum_k |product_k| elementwise (NaN/inf positions must agree)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), fin)
    with np.errstate(invalid="ignore"):  # (inf - inf at positions that are compared as a class above)
        err = np.abs(got - want)[fin]
    tol = rel * np.asarray(sum_abs, np.float64)[fin] + 1e-30
    bad = err > tol
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside {rel} * sum|p|; worst ratio {np.max(err / tol):.3g}"
