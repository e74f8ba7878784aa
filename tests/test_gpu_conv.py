"""AMConv2D forward / grad-input / grad-filter on the GPU (through the C ABI)
against the CPU oracle and, with the exact-on-integers ACC_7 table, against a
library convolution and its autograd (bit for bit)."""
import numpy as np
import pytest

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, asym_lut_u8, dev, host, lut32
from tests.util import REF_CONV_SHAPES, lut_path, small_ints, torch_conv_reference

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("amsim_engine")]


@pytest.fixture(scope="module")
def amd():
    import approxtrain_amd
    from approxtrain_amd import functors
    yield functors
    approxtrain_amd.load_library().amsim_set_split_k(1)


def _set_split(mode):
    import approxtrain_amd
    approxtrain_amd.load_library().amsim_set_split_k(mode)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("padding", ["VALID", "SAME"])
@pytest.mark.parametrize("shape", REF_CONV_SHAPES)
def test_conv_exact_against_library_conv(amd, shape, stride, padding):
    """The reference's own test design (test/convam_final_test.py): integer
    operands in [-2, 2), every shape x stride 1, 2 x VALID, SAME."""
    from approxtrain_amd import ApproxMulLut
    n, h, w_, c, kh, kw, _, oc = shape
    if padding == "VALID" and (kh > h or kw > w_):
        pytest.skip("empty VALID output")
    n = min(n, 16)
    _set_split(1)
    lut = ApproxMulLut.cached(lut_path("ACC", 7))
    rng = np.random.default_rng(abs(hash(shape)) % 1000 + stride)
    x, w = small_ints(rng, (n, h, w_, c), -2, 2), small_ints(rng, (kh, kw, c, oc), -2, 2)
    y = host(amd.convam(lut, dev(x), dev(w), (stride, stride), padding))
    dy = small_ints(rng, y.shape, -2, 2)
    y_ref, dx_ref, dw_ref = torch_conv_reference(x, w, dy, (stride, stride), padding)
    assert y.shape == y_ref.shape
    assert np.array_equal(y.astype(np.float64), y_ref)
    dx = host(amd.convam_input_grad(lut, x.shape, dev(w), dev(dy), (stride, stride), padding))
    dw = host(amd.convam_filter_grad(lut, dev(x), w.shape, dev(dy), (stride, stride), padding))
    assert np.array_equal(dx.astype(np.float64), dx_ref)
    assert np.array_equal(dw.astype(np.float64), dw_ref)


CASES = [
    # (x shape, w shape, stride, padding)
    ((2, 12, 12, 64), (3, 3, 64, 64), 1, "SAME"),     # the 3x3 ResNet layer, small image
    ((3, 9, 7, 32), (3, 3, 32, 48), 2, "SAME"),
    ((2, 14, 14, 6), (5, 5, 6, 16), 1, "VALID"),      # LeNet-5 conv2
    ((4, 28, 28, 1), (5, 5, 1, 6), 1, "SAME"),        # LeNet-5 conv1
    ((2, 8, 8, 16), (1, 1, 16, 24), 1, "VALID"),      # 1x1
    ((2, 6, 6, 8), (6, 6, 8, 10), 1, "VALID"),        # full-window
    ((1, 11, 13, 5), (4, 3, 5, 7), 3, "SAME"),
    ((8, 8, 8, 128), (1, 1, 128, 320), 1, "VALID"),   # few pixels, many channels (late ResNet stages): the
    ((4, 8, 8, 96), (3, 3, 96, 128), 1, "SAME"),      # reduction-slice arrangement under the LDS-table engine
    ((4, 16, 16, 64), (1, 1, 64, 160), 2, "VALID"),   # ... and a strided 1x1 (three pixel classes in four unreached)
]


@pytest.mark.parametrize("xs,ws,stride,padding", CASES)
def test_conv_against_oracle_real_multiplier(amd, xs, ws, stride, padding):
    from approxtrain_amd import ApproxMulLut
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    rng = np.random.default_rng(sum(xs) + sum(ws) + stride)
    x = np.maximum(rng.standard_normal(xs), 0).astype(np.float32)
    w = (rng.standard_normal(ws) * np.sqrt(2.0 / (ws[0] * ws[1] * ws[2]))).astype(np.float32)
    st = (stride, stride)
    want_y = cpu.conv2d_fwd(L, 7, x, w, st, padding)
    dy = rng.standard_normal(want_y.shape).astype(np.float32)
    want_dx = cpu.conv2d_grad_input(L, 7, xs, w, dy, st, padding)
    want_dw = cpu.conv2d_grad_filter(L, 7, x, ws, dy, st, padding)
    # unsplit: one ascending chain per output, bit-equal to the oracle
    _set_split(0)
    assert np.array_equal(host(amd.convam(lut, dev(x), dev(w), st, padding)).view(np.uint32), want_y.view(np.uint32))
    assert np.array_equal(host(amd.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding)).view(np.uint32),
                          want_dx.view(np.uint32))
    assert np.array_equal(host(amd.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding)).view(np.uint32),
                          want_dw.view(np.uint32))
    # default (split-K where it pays): within 1e-5 * sum|p|
    _set_split(1)
    abs_x, abs_w, abs_dy = np.abs(x), np.abs(w), np.abs(dy)
    # sum|p| <= exact conv of absolute values * (1 + 2^-7 headroom of the multiplier)
    s_y, s_dx, s_dw = torch_conv_reference(abs_x, abs_w, abs_dy, st, padding)
    assert_close_sum_abs(host(amd.convam(lut, dev(x), dev(w), st, padding)), want_y, s_y)
    assert_close_sum_abs(host(amd.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding)), want_dx, s_dx)
    assert_close_sum_abs(host(amd.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding)), want_dw, s_dw)


def test_conv_operand_order_asymmetric_lut(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    tab = asym_lut_u8(3)
    lut = ApproxMulLut.from_entries(tab, 3)
    L = cpu.expand_u8(tab, 3)
    rng = np.random.default_rng(71)
    xs, ws = (2, 7, 6, 5), (3, 2, 5, 9)
    x, w = rng.standard_normal(xs).astype(np.float32), rng.standard_normal(ws).astype(np.float32)
    y = cpu.conv2d_fwd(L, 3, x, w, (1, 1), "SAME")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    assert np.array_equal(host(amd.convam(lut, dev(x), dev(w), (1, 1), "SAME")).view(np.uint32), y.view(np.uint32))
    assert np.array_equal(host(amd.convam_input_grad(lut, xs, dev(w), dev(dy), (1, 1), "SAME")).view(np.uint32),
                          cpu.conv2d_grad_input(L, 3, xs, w, dy, (1, 1), "SAME").view(np.uint32))
    assert np.array_equal(host(amd.convam_filter_grad(lut, dev(x), ws, dev(dy), (1, 1), "SAME")).view(np.uint32),
                          cpu.conv2d_grad_filter(L, 3, x, ws, dy, (1, 1), "SAME").view(np.uint32))


def test_conv_special_values_in_input(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    lut = ApproxMulLut.cached(lut_path("MIT", 7))
    L = lut32("MIT", 7)
    rng = np.random.default_rng(72)
    xs, ws = (1, 6, 6, 32), (3, 3, 32, 16)
    x = rng.standard_normal(xs).astype(np.float32)
    w = rng.standard_normal(ws).astype(np.float32)
    x[0, 2, 3, 5] = np.inf; x[0, 0, 0, 0] = np.float32(1e-42); x[0, 5, 5, 31] = np.float32(1e30)
    w[1, 1, 7, 3] = np.float32(1e-39); w[0, 2, 9, 1] = np.float32(-2e30)
    with np.errstate(all="ignore"):
        want = cpu.conv2d_fwd(L, 7, x, w, (1, 1), "SAME")
    got = host(amd.convam(lut, dev(x), dev(w), (1, 1), "SAME"))
    both_nan = np.isnan(got) & np.isnan(want)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | both_nan).all()
