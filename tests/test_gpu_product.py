"""Elementwise approximate product on the GPU (through amsim_mul_f32) against
the CPU oracle: bit-exact over every mantissa pair x exponents x signs,
including zeros, subnormals, infinities and NaNs (NaNs compared as a class)."""
import os

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.util import GOLDEN, LUT_FILES, lut_bytes, lut_path, product_domain, same_bits_or_both_nan

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_product_bit_exact_full_domain(kind, m):
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut(lut_path(kind, m))
    assert lut.mant_width == m
    a, b = product_domain(m, seed=400 + m)
    af, bf = a.view(np.float32), b.view(np.float32)
    got = functors.mul(lut, torch.from_numpy(af).cuda(), torch.from_numpy(bf).cuda()).cpu().numpy()
    want = cpu.lut_mul_array(cpu.expand_u8(lut_bytes(kind, m), m), m, af, bf)
    ok = same_bits_or_both_nan(got, want)
    assert ok.all(), f"{(~ok).sum()} mismatches of {ok.size}; first {np.flatnonzero(~ok)[:5]}"


def test_product_against_reference_model_vectors():
    """Golden vectors written by the reference's own compiled C models
    (tests/golden/make_product_vectors.py)."""
    from approxtrain_amd import ApproxMulLut, functors
    path = os.path.join(GOLDEN, "product_vectors.npz")
    data = np.load(path, allow_pickle=False)
    for kind, m in LUT_FILES:
        if kind == "ACC":
            continue
        a, b, want = data[f"{kind}_{m}_a"], data[f"{kind}_{m}_b"], data[f"{kind}_{m}_out"]
        lut = ApproxMulLut(lut_path(kind, m))
        got = functors.mul(lut, torch.from_numpy(a.view(np.float32)).cuda(),
                           torch.from_numpy(b.view(np.float32)).cuda()).cpu().numpy()
        ok = same_bits_or_both_nan(got, want.view(np.float32))
        assert ok.all(), f"{kind}_{m}: {(~ok).sum()} mismatches"


def test_product_m11_legacy_entries():
    """32-bit legacy entries (bit 31 carry, mantissa in place) at m = 11."""
    from approxtrain_amd import ApproxMulLut, functors
    m = 11
    img = cpu.lutgen32("MIT", m)  # carry<<23 | mant<<(23-m)
    legacy = ((img >> 23) << 31) | (img & 0x7fffff)
    lut = ApproxMulLut.from_entries(legacy.astype(np.uint32), m)
    rng = np.random.default_rng(7)
    a = rng.standard_normal(1 << 18).astype(np.float32)
    b = rng.standard_normal(1 << 18).astype(np.float32)
    got = functors.mul(lut, torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()).cpu().numpy()
    want = cpu.lut_mul_array(img, m, a, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _exhaustive_sweep(kind, m, bits, block):
    """GPU product (amsim_mul_f32) against the oracle's LUT product over ALL pairs of the 2^bits
    (sign, exponent, m-bit mantissa) operand patterns, low fraction bits zero: the design of the
    reference's own sweep (lut/test.cc:41-107), without its exclusion of zero-exponent operands.
    Operands are generated on the device, block by block; the oracle runs on host threads."""
    from concurrent.futures import ThreadPoolExecutor
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut(lut_path(kind, m))
    lut32 = cpu.expand_u8(lut_bytes(kind, m), m)
    shift = 32 - bits
    n = 1 << bits
    j_dev = (torch.arange(n, dtype=torch.int64, device="cuda") << shift).to(torch.int32)  # wraps into the sign bit
    workers = min(16, cpu.max_threads())
    total = bad = 0

    def oracle(args):
        a, b = args
        return cpu.lut_mul_array(lut32, m, a, b)

    with ThreadPoolExecutor(max_workers=workers) as pool:
        for i0 in range(0, n, block):
            i_dev = (torch.arange(i0, i0 + block, dtype=torch.int64, device="cuda") << shift).to(torch.int32)
            a_dev = i_dev.repeat_interleave(n).view(torch.float32)
            b_dev = j_dev.repeat(block).view(torch.float32)
            got = functors.mul(lut, a_dev, b_dev).cpu().numpy()
            a, b = a_dev.cpu().numpy(), b_dev.cpu().numpy()
            parts = np.array_split(np.arange(a.size), workers)
            want = np.concatenate(list(pool.map(oracle, [(a[p[0]:p[-1] + 1], b[p[0]:p[-1] + 1]) for p in parts])))
            bad += int((~same_bits_or_both_nan(got, want)).sum())
            total += a.size
    assert total == 1 << (2 * bits)
    assert bad == 0, f"{kind}_{m}: {bad} of {total} products differ from the oracle"


@pytest.mark.parametrize("kind", ["MBM", "MIT"])
def test_exhaustive_top_bit_patterns_width5(kind):
    """All 2^14 x 2^14 = 2^28 pairs of (sign, exponent, 5-bit mantissa) patterns."""
    _exhaustive_sweep(kind, 5, 14, 1 << 10)


@pytest.mark.parametrize("kind", ["MBM", "MIT"])
def test_exhaustive_top_bit_patterns_width7(kind):
    """All 2^16 x 2^16 = 2^32 pairs of (sign, exponent, 7-bit mantissa) patterns: every operand
    the truncating multiplier can tell apart, crossed with every other one."""
    _exhaustive_sweep(kind, 7, 16, 1 << 10)
