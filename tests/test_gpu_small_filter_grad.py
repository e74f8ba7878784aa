"""Filter gradients of small layers (few filter elements x output channels, many pixels) on the
kernel that spreads the REDUCTION over the lanes: through the C ABI, against the CPU oracle's loop
nest (cuda/cuda_kernel.cu:327-353 + cuda/gemm.cu:17-58).  That kernel adds each output's products
in a fixed order that is not one ascending chain, so it only serves calls whose reductions may be
split: results within 1e-5 * sum|products| of the sequential oracle and identical from run to run;
the same calls through a whole-reduction handle stay bit-equal to the oracle (other engines)."""
import numpy as np
import pytest

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, dev, host, lut32
from tests.util import lut_path, torch_conv_reference

pytestmark = pytest.mark.gpu


def _handles(kind, m):
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    split, whole = ApproxMulLut(lut_path(kind, m)), ApproxMulLut(lut_path(kind, m))
    assert lib.amsim_lut_set_split_k(split.handle, 1) == 0 and lib.amsim_lut_set_split_k(whole.handle, 0) == 0
    return split, whole, lut32(kind, m)


def _check(kind, m, x, ws, dy, st, padding):
    from approxtrain_amd import functors
    split, whole, L = _handles(kind, m)
    want = cpu.conv2d_grad_filter(L, m, x, ws, dy, st, padding, threads=cpu.max_threads())
    sum_abs = torch_conv_reference(np.abs(np.nan_to_num(x, nan=0.0, posinf=0.0, neginf=0.0)), np.zeros(ws, np.float32),
                                   np.abs(dy), st, padding)[2] * 1.01
    got = host(functors.convam_filter_grad(split, dev(x), ws, dev(dy), st, padding))
    assert_close_sum_abs(got, want, sum_abs)
    again = host(functors.convam_filter_grad(split, dev(x), ws, dev(dy), st, padding))
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    exact = host(functors.convam_filter_grad(whole, dev(x), ws, dev(dy), st, padding))
    fin = np.isfinite(want)
    assert np.array_equal(exact.view(np.uint32)[fin], want.view(np.uint32)[fin]) and np.array_equal(np.isnan(exact), np.isnan(want))


@pytest.mark.parametrize("kind,m", [("MIT", 7), ("MBM", 7), ("MBM", 3)])
@pytest.mark.parametrize("xs,ws,padding", [((256, 28, 28, 1), (5, 5, 1, 6), "SAME"),     # LeNet-5 conv1
                                           ((256, 14, 14, 6), (5, 5, 6, 16), "VALID")])   # LeNet-5 conv2
def test_lenet5_filter_gradients(kind, m, xs, ws, padding):
    rng = np.random.default_rng(m + xs[1])
    x = np.abs(rng.standard_normal(xs)).astype(np.float32) * (rng.random(xs) > 0.2)
    oh = xs[1] if padding == "SAME" else xs[1] - ws[0] + 1
    dy = (rng.standard_normal((xs[0], oh, oh, ws[3])) * 0.1).astype(np.float32)
    _check(kind, m, x, ws, dy, (1, 1), padding)


@pytest.mark.parametrize("seed", range(16))
def test_random_small_filter_gradients(seed):
    """Odd extents, strides, paddings, channel counts, block shapes with and without padding; a third
    of the cases carry values outside the fast product's range (subnormal, tiny, huge, infinite, NaN)
    in the input, which send their 64-pixel passes through the full-domain product."""
    rng = np.random.default_rng(600 + seed)
    c = int(rng.choice([1, 2, 3, 6, 8]))
    oc = int(rng.choice([1, 3, 6, 8, 11, 16]))
    kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    st = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    padding = str(rng.choice(["SAME", "VALID"]))
    n, h, w = int(rng.integers(8, 40)), int(rng.integers(kh + 10, kh + 26)), int(rng.integers(kw + 10, kw + 26))
    xs, ws = (n, h, w, c), (kh, kw, c, oc)
    x = rng.standard_normal(xs).astype(np.float32) * (rng.random(xs) > 0.3)
    if seed % 3 == 2:
        hit = rng.random(xs) < 0.001
        x[hit] = rng.choice(np.array([1e-40, -1e-42, 1e-30, 2e-38, 1e30, -3e30, np.inf, np.nan], np.float32), size=int(hit.sum()))
    L = lut32("MBM", 7)
    y_shape = cpu.conv2d_fwd(L, 7, np.zeros(xs, np.float32), np.zeros(ws, np.float32), st, padding).shape
    dy = rng.standard_normal(y_shape).astype(np.float32) * (rng.random(y_shape) > 0.1)
    kind, m = [("MBM", 7), ("MIT", 7), ("MIT", 5), ("MBM", 1)][seed % 4]
    _check(kind, m, x, ws, dy, st, padding)


@pytest.mark.parametrize("sx,sdy", [(0, -80), (-30, -70), (-90, -60), (40, 50), (110, 60)])
def test_far_off_exponents(sx, sdy):
    """Gradients (and inputs) scaled far outside the quick test's exponent interval: the pass still
    takes the fast product form when the two exponent ranges allow it, the full-domain product when
    products would under- or overflow; checked against the oracle at the usual tolerance."""
    from approxtrain_amd import functors
    rng = np.random.default_rng(abs(sx) + 3 * abs(sdy))
    xs, ws = (64, 20, 20, 1), (5, 5, 1, 6)
    x = (rng.standard_normal(xs) * 2.0 ** sx).astype(np.float32)
    dy = (rng.standard_normal((64, 20, 20, 6)) * 2.0 ** sdy).astype(np.float32)
    split, whole, L = _handles("MIT", 7)
    want = cpu.conv2d_grad_filter(L, 7, x, ws, dy, (1, 1), "SAME", threads=cpu.max_threads()).astype(np.float64)
    got = host(functors.convam_filter_grad(split, dev(x), ws, dev(dy), (1, 1), "SAME")).astype(np.float64)
    exact = host(functors.convam_filter_grad(whole, dev(x), ws, dev(dy), (1, 1), "SAME"))
    assert np.array_equal(exact.view(np.uint32), want.astype(np.float32).view(np.uint32))
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    scale = np.abs(want[np.isfinite(want)]).max() if np.isfinite(want).any() else 0.0
    fin = np.isfinite(want)
    assert np.all(np.abs(got - want)[fin] <= 2e-4 * scale + 1e-45)   # 6400 products per output, partial sums in another order
