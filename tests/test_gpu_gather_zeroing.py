"""The LDS-table GEMM gathers table bytes into the upper half of registers whose lower half must
read as zero.  Devices differ in what a 16-bit LDS load does to the other half (kept or cleared):
the library probes this once per device and, where the half is kept, zeroes the registers once per
reduction chunk.  Here that branch is forced on (amsim_lut_force_gather_zeroing), whatever the
probe said: results must be the oracle's, bit for bit, for every operand source of the engine
(dense in both layouts, convolution patches, filter-gradient gather), every column-tile width and
with operands that take the full-domain path."""
import ctypes as C

import numpy as np
import pytest

import approxtrain_amd
from oracle import cpu
from tests.gpu_util import dev, host, lut32
from tests.util import lut_path, same_bits_or_both_nan

pytestmark = pytest.mark.gpu


def _handle(forced):
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut(lut_path("MBM", 7))
    probed = C.c_int(-1)
    assert lib.amsim_lut_set_split_k(lut.handle, 0) == 0   # whole reductions: bit-equal to the oracle
    assert lib.amsim_lut_set_engine(lut.handle, 1) == 0    # the LDS-table engine
    assert lib.amsim_lut_force_gather_zeroing(lut.handle, 1 if forced else 0, C.byref(probed)) == 0
    assert probed.value in (0, 1)
    return lut


def test_the_probe_has_an_answer_and_the_hook_checks_its_arguments():
    lib = approxtrain_amd.load_library()
    lut = _handle(False)
    assert lib.amsim_lut_force_gather_zeroing(lut.handle, 2, None) != 0
    assert lib.amsim_lut_force_gather_zeroing(None, 1, None) != 0
    assert lib.amsim_lut_force_gather_zeroing(lut.handle, 1, None) == 0
    lut.close()


@pytest.mark.parametrize("forced", [True, False])
@pytest.mark.parametrize("ta,tb,M,N,K", [(0, 0, 300, 70, 100), (1, 0, 257, 64, 333), (0, 1, 130, 9, 96), (1, 1, 64, 2, 50),
                                          (0, 0, 1000, 24, 64), (0, 0, 200, 1, 40), (0, 0, 2048, 6, 200)])
def test_gemm_with_forced_zeroing(forced, ta, tb, M, N, K):
    from approxtrain_amd import functors
    lut, L = _handle(forced), lut32("MBM", 7)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    A[rng.random(A.shape) < 0.15] = 0.0
    B.flat[::37] = np.float32(1e-42)   # subnormals: those chunks take the full-domain product
    A.flat[5::53] = np.float32(np.inf)
    got = host(functors.gemm(lut, dev(A), dev(B), trans_a=bool(ta), trans_b=bool(tb)))
    want = cpu.gemm(L, 7, A, B, transA=bool(ta), transB=bool(tb), threads=8)
    assert np.all(same_bits_or_both_nan(got, want))
    lut.close()


@pytest.mark.parametrize("forced", [True, False])
@pytest.mark.parametrize("xs,ws,stride,padding", [((2, 14, 14, 32), (3, 3, 32, 48), 1, "SAME"), ((3, 9, 11, 5), (3, 2, 5, 7), 2, "VALID"),
                                                  ((2, 8, 8, 64), (1, 1, 64, 32), 1, "SAME")])
def test_convolution_passes_with_forced_zeroing(forced, xs, ws, stride, padding):
    from approxtrain_amd import functors
    lut, L = _handle(forced), lut32("MBM", 7)
    rng = np.random.default_rng(sum(xs) + sum(ws))
    x = np.maximum(rng.standard_normal(xs), 0).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.1).astype(np.float32)
    y = cpu.conv2d_fwd(L, 7, x, w, (stride, stride), padding)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    got = host(functors.convam(lut, dev(x), dev(w), (stride, stride), padding))
    assert np.array_equal(got.view(np.uint32), y.view(np.uint32))
    gi = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), (stride, stride), padding))
    assert np.array_equal(gi.view(np.uint32), cpu.conv2d_grad_input(L, 7, xs, w, dy, (stride, stride), padding).view(np.uint32))
    gf = host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), (stride, stride), padding))
    assert np.array_equal(gf.view(np.uint32), cpu.conv2d_grad_filter(L, 7, x, ws, dy, (stride, stride), padding).view(np.uint32))
    lut.close()
