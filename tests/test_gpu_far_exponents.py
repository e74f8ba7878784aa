"""Operands far outside the quick test's exponent interval [2^-63, 2^64): tiny gradients times
ordinary weights and the like.  The engines take a second look at such chunks -- the two operands'
exponent ranges decide whether every product can still use the fast form -- and fall back to the
full-domain product only where products would under- or overflow.  Whatever path runs, the result
is bit-equal to the CPU oracle's loop nests (reductions kept whole), under every engine setting."""
import numpy as np
import pytest

from oracle import cpu
from tests.gpu_util import dev, host, lut32
from tests.util import lut_path, same_bits_or_both_nan

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("amsim_engine")]

SCALES = [(0, -80), (-85, 0), (-60, -60), (-70, -57), (-100, -30), (90, 30), (100, 27), (120, 10), (-126, 0), (-20, 127)]


def _lut():
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lut = ApproxMulLut(lut_path("MBM", 7))
    assert approxtrain_amd.load_library().amsim_lut_set_split_k(lut.handle, 0) == 0
    return lut, lut32("MBM", 7)


@pytest.mark.parametrize("sa,sb", SCALES)
@pytest.mark.parametrize("shape", [(300, 70, 100), (64, 5, 40), (1000, 24, 333)])
def test_gemm(sa, sb, shape):
    from approxtrain_amd import functors
    lut, L = _lut()
    M, N, K = shape
    rng = np.random.default_rng(abs(sa) + 5 * abs(sb) + M)
    with np.errstate(over="ignore"):  # (the largest scale sends some elements to infinity: on purpose)
        A = (rng.standard_normal((M, K)) * 2.0 ** sa).astype(np.float32) * (rng.random((M, K)) > 0.1)
        B = (rng.standard_normal((K, N)) * 2.0 ** sb).astype(np.float32)
    got = host(functors.gemm(lut, dev(A), dev(B)))
    assert np.all(same_bits_or_both_nan(got, cpu.gemm(L, 7, A, B)))


@pytest.mark.parametrize("sa,sb", [(0, 0), (0, -80), (-85, 0), (-60, -60), (-70, -57), (-100, -30), (40, 40)])
def test_gemm_with_split_reductions(sa, sb, amsim_engine):
    """One row tile, three column groups, a long reduction, reductions free to be split: under the
    LDS-table engine the reduction rows of every chunk are dealt out to a workgroup's four wavefronts
    (and the chunks to many workgroups), so the second look and the full-domain products run inside
    that arrangement too.  Within 1e-5 * sum|products| of the oracle's sequential chain."""
    import ctypes as C
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    from tests.gpu_util import assert_close_sum_abs
    lib = approxtrain_amd.load_library()
    M, N, K = 64, 40, 2000
    if amsim_engine == "lds_table":
        info = (C.c_int64 * 8)()
        assert lib.amsim_gemm_plan_info(0, 0, M, N, K, 1, info) == 0
        assert info[1] == 0, list(info)  # the reduction-slice arrangement
    lut, L = ApproxMulLut(lut_path("MBM", 7)), lut32("MBM", 7)
    rng = np.random.default_rng(abs(sa) + 7 * abs(sb))
    A = (rng.standard_normal((M, K)) * 2.0 ** sa).astype(np.float32) * (rng.random((M, K)) > 0.1)
    B = (rng.standard_normal((K, N)) * 2.0 ** sb).astype(np.float32)
    got = host(functors.gemm(lut, dev(A), dev(B)))
    assert_close_sum_abs(got, cpu.gemm(L, 7, A, B), cpu.gemm_abs(L, 7, A, B), 1e-5)


@pytest.mark.parametrize("sx,sw,sdy", [(0, 0, -80), (0, -10, -100), (-40, -50, -30), (30, 40, 50), (0, 0, 100)])
def test_convolution_passes(sx, sw, sdy):
    from approxtrain_amd import functors
    lut, L = _lut()
    rng = np.random.default_rng(abs(sx) + abs(sw) + abs(sdy))
    xs, ws = (3, 17, 19, 8), (3, 3, 8, 12)
    x = (np.maximum(rng.standard_normal(xs), 0) * 2.0 ** sx).astype(np.float32)
    w = (rng.standard_normal(ws) * 2.0 ** sw).astype(np.float32)
    y = cpu.conv2d_fwd(L, 7, x, w, (1, 1), "SAME")
    dy = (rng.standard_normal(y.shape) * 2.0 ** sdy).astype(np.float32)
    assert np.all(same_bits_or_both_nan(host(functors.convam(lut, dev(x), dev(w), (1, 1), "SAME")), y))
    assert np.all(same_bits_or_both_nan(host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), (1, 1), "SAME")),
                                        cpu.conv2d_grad_input(L, 7, xs, w, dy, (1, 1), "SAME")))
    assert np.all(same_bits_or_both_nan(host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), (1, 1), "SAME")),
                                        cpu.conv2d_grad_filter(L, 7, x, ws, dy, (1, 1), "SAME")))
