"""A bounded, seeded sweep over the work planner's decisions for the LDS-table GEMM engine.

The planner shapes a problem as workgroups over row tiles x column groups, optionally with the
reduction split across workgroups (partial sums added by a reduction pass), with a split "tail"
for the rows of a mostly empty last round, or with the reduction rows of each chunk dealt out to
the four wavefronts of a workgroup ("slices").  Which of these a shape gets is asked from the
library itself (amsim_gemm_plan_info), candidates come from a seeded stream, and a few shapes of
every kind of plan met are kept -- so the sweep follows the planner when its rules change.

Every kept shape runs on the GPU through the C ABI with the direct engine switched off (so the
planner's path is the one that runs), once with split reductions allowed (within
1e-5 * sum|products| of the oracle, and identical on a second run) and once with reductions
kept whole (bit-equal to the oracle's sequential chains)."""
import ctypes as C

import numpy as np
import pytest

import approxtrain_amd
from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, dev, host, lut32
from tests.util import lut_path

pytestmark = pytest.mark.gpu
REL = 1e-5
PER_KIND = 4
MAX_MACS = 2.5e8
MAX_MACS_LARGE = 1.0e9  # the few many-row shapes that reach tails and plain splits
THREADS = 16


def plan_of(lib, ta, tb, M, N, K):
    info = (C.c_int64 * 8)()
    assert lib.amsim_gemm_plan_info(ta, tb, M, N, K, 1, info) == 0
    tn, wr, nsplit, _, _, tail_nsplit, _, nchunks = list(info)
    kind = ("slices" if wr == 0 else "four-row-tiles" if wr == 4 else "one-row-tile",
            "split" if nsplit > 1 else "whole", "tail" if tail_nsplit > 0 else "no-tail", tn)
    return kind, nchunks


def sweep_shapes():
    lib = approxtrain_amd.load_library()
    rng = np.random.default_rng(5)
    kept, kinds = [], {}
    # large-row problems first (tails and plain splits need many row tiles), then the general stream
    stream = [(int(rng.integers(0, 2)), int(rng.integers(0, 2)), int(m * rng.uniform(0.8, 1.25)), n, k)
              for m, n, k in ((100352, 64, 128), (100000, 64, 96), (25088, 128, 256), (50176, 64, 128), (6272, 256, 288),
                              (12544, 128, 96), (6179, 100, 576), (13705, 40, 576), (25000, 64, 150), (3571, 512, 100),
                              (1568, 512, 320))
              for _ in range(6)]
    n_large = len(stream)
    for _ in range(3000):
        m = int(rng.choice([64, 100, 256, 700, 1500, 3000, 6000, 12000, 20000]) * rng.uniform(0.7, 1.3))
        n = int(rng.choice([1, 2, 3, 6, 8, 16, 40, 64, 100, 128, 256, 512]))
        k = int(rng.choice([32, 64, 100, 256, 576, 1000, 2304, 4608]))
        stream.append((int(rng.integers(0, 2)), int(rng.integers(0, 2)), m, n, k))
    for i, (ta, tb, m, n, k) in enumerate(stream):
        if m * n * k > (MAX_MACS_LARGE if i < n_large else MAX_MACS):
            continue
        kind, _ = plan_of(lib, ta, tb, m, n, k)
        if len(kinds.setdefault(kind, [])) < PER_KIND:
            kinds[kind].append((ta, tb, m, n, k))
            kept.append((ta, tb, m, n, k, kind))
    return kept


SHAPES = sweep_shapes()


def test_the_sweep_meets_every_kind_of_plan():
    kinds = {s[5] for s in SHAPES}
    assert 40 <= len(SHAPES) <= 90, len(SHAPES)
    assert {k[0] for k in kinds} >= {"one-row-tile", "four-row-tiles"}
    assert {k[1] for k in kinds} == {"whole", "split"}
    assert any(k[2] == "tail" for k in kinds), "no shape with a split tail"


@pytest.mark.parametrize("ta,tb,M,N,K,kind", SHAPES, ids=["%s-%s-%s-tn%d-%dx%dx%d-%d%d" % (s[5][:3] + (s[5][3], s[2], s[3], s[4], s[0], s[1])) for s in SHAPES])
def test_planned_gemm_matches_the_oracle_in_both_split_modes(ta, tb, M, N, K, kind):
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    L = lut32("MBM", 7)
    rng = np.random.default_rng(M * 31 + N * 7 + K)
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    A[rng.random(A.shape) < 0.2] = 0.0  # zeros take the all-zero table row / the zero multiplier
    want = cpu.gemm(L, 7, A, B, transA=bool(ta), transB=bool(tb), threads=THREADS)
    sum_abs = cpu.gemm_abs(L, 7, A, B, transA=bool(ta), transB=bool(tb), threads=THREADS)
    Ad, Bd = dev(A), dev(B)
    lut = ApproxMulLut(lut_path("MBM", 7))  # handles of this test's own: engine and split mode are per handle
    try:
        assert lib.amsim_lut_set_engine(lut.handle, 1) == 0  # LDS-table engine: the planner's path
        assert lib.amsim_lut_set_split_k(lut.handle, 1) == 0
        got = host(functors.gemm(lut, Ad, Bd, trans_a=bool(ta), trans_b=bool(tb)))
        assert_close_sum_abs(got, want, sum_abs, REL)
        again = host(functors.gemm(lut, Ad, Bd, trans_a=bool(ta), trans_b=bool(tb)))
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), "split reductions must be reproducible"
        assert lib.amsim_lut_set_split_k(lut.handle, 0) == 0
        whole = host(functors.gemm(lut, Ad, Bd, trans_a=bool(ta), trans_b=bool(tb)))
        assert np.array_equal(whole.view(np.uint32), want.view(np.uint32)), "whole reductions are the oracle's chains"
    finally:
        lut.close()
