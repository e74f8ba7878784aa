"""Seeded random sweep over convolution and GEMM shapes (odd extents, channel counts that are
and are not multiples of 4 / 32 / 64, strides 1-3, both paddings, transposes, batches): the three
convolution passes and the GEMM against the CPU oracle -- bit for bit with reductions kept
whole, within 1e-5 * sum|products| when the planner may split them.  Half of the whole-reduction
cases carry a sprinkle of special values (inf, NaN, subnormals, huge, tiny, signed zeros) in
every operand; NaN results are compared as a class."""
import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, dev, host, lut32
from tests.util import lut_path, same_bits_or_both_nan

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("amsim_engine")]


SPECIALS = np.array([np.inf, -np.inf, np.nan, 1e-40, -1e-42, 3e38, -3e38, 1e-30, 2e-38, 0.0, -0.0], dtype=np.float32)


def _spice(rng, a, p):
    """Replaces a fraction p of the elements by special values."""
    if p <= 0:
        return a
    hit = rng.random(a.shape) < p
    a = a.copy()
    a[hit] = rng.choice(SPECIALS, size=int(hit.sum()))
    return a


def _conv_case(rng):
    c = int(rng.choice([1, 3, 4, 6, 8, 16, 32, 64, 96]))
    oc = int(rng.choice([1, 2, 5, 8, 16, 24, 64, 80]))
    kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    h, w = int(rng.integers(kh, kh + 14)), int(rng.integers(kw, kw + 14))
    n = int(rng.integers(1, 5))
    st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    return (n, h, w, c), (kh, kw, c, oc), st, str(rng.choice(["SAME", "VALID"]))


@pytest.mark.parametrize("seed", range(40))
@pytest.mark.parametrize("split", [0, 1])
def test_random_convolutions(seed, split):
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(split)
    try:
        rng = np.random.default_rng(1000 + seed)
        xs, ws, st, padding = _conv_case(rng)
        kind = str(rng.choice(["MBM", "MIT"]))
        lut, L = ApproxMulLut.cached(lut_path(kind, 7)), lut32(kind, 7)
        p = (0.0, 0.0, 0.002, 0.02)[seed % 4] if split == 0 else 0.0
        x = _spice(rng, rng.standard_normal(xs).astype(np.float32) * (rng.random(xs) > 0.3), p)   # some exact zeros
        w = _spice(rng, rng.standard_normal(ws).astype(np.float32), p)
        want_y = cpu.conv2d_fwd(L, 7, x, w, st, padding)
        if want_y.size == 0:
            pytest.skip("empty output")
        dy = _spice(rng, rng.standard_normal(want_y.shape).astype(np.float32), p)
        got = [host(functors.convam(lut, dev(x), dev(w), st, padding)),
               host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding)),
               host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding))]
        want = [want_y, cpu.conv2d_grad_input(L, 7, xs, w, dy, st, padding),
                cpu.conv2d_grad_filter(L, 7, x, ws, dy, st, padding)]
        for g, v in zip(got, want):
            if split == 0:
                assert np.all(same_bits_or_both_nan(g, v)), (xs, ws, st, padding)
            else:
                scale = 1e-5 * (np.abs(v).max() * 64 + 1.0)
                assert np.all(np.abs(g - v) <= scale), (xs, ws, st, padding)
    finally:
        lib.amsim_set_split_k(1)


@pytest.mark.parametrize("seed", range(36))
def test_random_gemms(seed):
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    rng = np.random.default_rng(2000 + seed)
    M, N, K = (int(v) for v in rng.integers(1, 200, 3))
    if seed % 3 == 0:
        K = int(rng.integers(500, 3000))
    nb = int(rng.choice([0, 0, 1, 3, 7]))            # 0: rank-2 operands; else a strided batch
    shared_b = bool(nb and seed % 2 == 0)            # every item uses the same second operand
    ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    p = (0.0, 0.0, 0.002, 0.02)[seed % 4]
    sa = ((nb,) if nb else ()) + ((K, M) if ta else (M, K))
    sb = ((nb,) if nb and not shared_b else ()) + ((N, K) if tb else (K, N))
    A = _spice(rng, rng.standard_normal(sa).astype(np.float32), p)
    B = _spice(rng, rng.standard_normal(sb).astype(np.float32), p)
    lut, L = ApproxMulLut.cached(lut_path("MBM", 7)), lut32("MBM", 7)

    def oracle(fn):
        if not nb:
            return fn(L, 7, A, B, transA=int(ta), transB=int(tb))
        return np.stack([fn(L, 7, A[i], B if B.ndim == 2 else B[i], transA=int(ta), transB=int(tb)) for i in range(nb)])

    want = oracle(cpu.gemm)
    lib.amsim_set_split_k(0)
    try:
        got = host(functors.gemm(lut, dev(A), dev(B), trans_a=ta, trans_b=tb))
        assert got.shape == want.shape and np.all(same_bits_or_both_nan(got, want)), (M, N, K, nb, ta, tb)
    finally:
        lib.amsim_set_split_k(1)
    if p == 0.0:
        got = host(functors.gemm(lut, dev(A), dev(B), trans_a=ta, trans_b=tb))
        assert_close_sum_abs(got, want, oracle(cpu.gemm_abs), 1e-5)
