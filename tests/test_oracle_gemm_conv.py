"""Pins the oracle's GEMM / dense / matmul / convolution loop nests by
mathematics: with a multiplier that is exact on the chosen operands (ACC_7 on
integers with <= 3 significant fraction bits, MIT on powers of two) every
result must equal exact integer arithmetic, i.e. a library matmul /
convolution and its autograd, bit for bit.  A wrong index, pad, stride, flip
or operand transposition fails.  CPU only."""
import numpy as np
import pytest

from oracle import cpu
from tests.util import REF_CONV_SHAPES, lut_bytes, small_ints, torch_conv_reference

ACC7 = cpu.expand_u8(lut_bytes("ACC", 7), 7)
MIT7 = cpu.expand_u8(lut_bytes("MIT", 7), 7)
MBM7 = cpu.expand_u8(lut_bytes("MBM", 7), 7)


def asym_lut(m=3):
    """A deliberately asymmetric table: entry depends on (ma, mb) order."""
    n = 1 << m
    i, j = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32), indexing="ij")
    return (((i * 3 + j * 5 + 1) % n) << (23 - m)).astype(np.uint32).ravel() | (((i > j).astype(np.uint32)) << 23).ravel()


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm_exact_against_integer_matmul(ta, tb):
    rng = np.random.default_rng(1)
    M, N, K = 37, 29, 53
    A = small_ints(rng, (K, M) if ta else (M, K))
    B = small_ints(rng, (N, K) if tb else (K, N))
    want = (A.T if ta else A).astype(np.int64) @ (B.T if tb else B).astype(np.int64)
    got = cpu.gemm(ACC7, 7, A, B, transA=ta, transB=tb)
    assert np.array_equal(got.astype(np.int64), want)
    got = cpu.gemm(ACC7, 7, A, B, transA=ta, transB=tb, swap=True)
    assert np.array_equal(got.astype(np.int64), want)


def test_gemm_mitchell_powers_of_two():
    rng = np.random.default_rng(2)
    A = (np.float32(2.0) ** rng.integers(-5, 6, (17, 40))) * rng.choice([-1, 1], (17, 40))
    B = (np.float32(2.0) ** rng.integers(-5, 6, (40, 9))) * rng.choice([-1, 1], (40, 9))
    want = A.astype(np.float64) @ B.astype(np.float64)
    got = cpu.gemm(MIT7, 7, A.astype(np.float32), B.astype(np.float32))
    assert np.array_equal(got.astype(np.float64), want)  # sums of dyadics < 2^24 are exact


def test_gemm_operand_order_and_accumulation_order():
    lut = asym_lut(3)
    rng = np.random.default_rng(3)
    A = rng.standard_normal((5, 11)).astype(np.float32)
    B = rng.standard_normal((11, 4)).astype(np.float32)
    got = cpu.gemm(lut, 3, A, B)
    got_sw = cpu.gemm(lut, 3, A, B, swap=True)
    want = np.zeros((5, 4), np.float32)
    want_sw = np.zeros((5, 4), np.float32)
    for i in range(5):
        for j in range(4):
            acc = np.float32(0)
            acc_sw = np.float32(0)
            for k in range(11):
                acc = np.float32(acc + cpu.lut_mul_array(lut, 3, A[i, k:k + 1], B[k:k + 1, j])[0])
                acc_sw = np.float32(acc_sw + cpu.lut_mul_array(lut, 3, B[k:k + 1, j], A[i, k:k + 1])[0])
            want[i, j], want_sw[i, j] = acc, acc_sw
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got_sw.view(np.uint32), want_sw.view(np.uint32))
    assert not np.array_equal(got, got_sw)  # the table really is asymmetric


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("swap", [False, True])
def test_gemm_abs_is_the_product_of_absolute_integer_matrices(ta, tb, swap):
    """The tolerance normaliser sum_k |P(a, b)|: with ACC_7 on small integers every product is
    exact, so the sum must equal |op(A)| . |op(B)| exactly for every transpose form and either
    operand order (a wrong index or transposition changes it; cancelling signs would too)."""
    rng = np.random.default_rng(21)
    M, N, K = 23, 31, 47
    A = small_ints(rng, (K, M) if ta else (M, K))
    B = small_ints(rng, (N, K) if tb else (K, N))
    want = np.abs(A.T if ta else A).astype(np.int64) @ np.abs(B.T if tb else B).astype(np.int64)
    got = cpu.gemm_abs(ACC7, 7, A, B, transA=ta, transB=tb, swap=swap)
    assert got.dtype == np.float64 and np.array_equal(got, want.astype(np.float64))
    # sum|p| >= |sum p|, with equality only where no signs cancel: the signed GEMM differs
    signed = cpu.gemm(ACC7, 7, A, B, transA=ta, transB=tb, swap=swap).astype(np.float64)
    assert np.all(got >= np.abs(signed)) and np.any(got > np.abs(signed))


def test_gemm_abs_sums_the_lut_products_and_skips_non_finite_ones():
    """With the real multiplier (MBM_7) and an asymmetric table: the sum of |lut_mul| of every
    operand pair, in float64; infinite and NaN products are left out (they are compared as a class)."""
    rng = np.random.default_rng(22)
    A = rng.standard_normal((6, 13)).astype(np.float32)
    B = rng.standard_normal((13, 5)).astype(np.float32)
    A[2, 3], B[4, 1] = np.inf, np.nan
    for lut, m in ((MBM7, 7), (asym_lut(3), 3)):
        for swap in (False, True):
            want = np.zeros((6, 5))
            for i in range(6):
                for j in range(5):
                    a, b = A[i], np.ascontiguousarray(B[:, j])
                    p = cpu.lut_mul_array(lut, m, b, a) if swap else cpu.lut_mul_array(lut, m, a, b)
                    p = p.astype(np.float64)
                    want[i, j] = np.abs(p[np.isfinite(p)]).sum()
            got = cpu.gemm_abs(lut, m, A, B, swap=swap)
            assert np.allclose(got, want, rtol=1e-14, atol=0)
    assert not np.array_equal(cpu.gemm_abs(asym_lut(3), 3, A, B), cpu.gemm_abs(asym_lut(3), 3, A, B, swap=True))


def test_dense_fwd_and_grads_exact():
    rng = np.random.default_rng(4)
    x, w, dy = small_ints(rng, (6, 13)), small_ints(rng, (13, 7)), small_ints(rng, (6, 7))
    assert np.array_equal(cpu.dense_fwd(ACC7, 7, x, w), x @ w)
    dx, dw = cpu.dense_grad(ACC7, 7, dy, x, w)
    assert np.array_equal(dx, dy @ w.T)
    assert np.array_equal(dw, x.T @ dy)


def test_dense_grad_x_feeds_weight_as_first_operand():
    lut = asym_lut(3)
    rng = np.random.default_rng(5)
    x, w, dy = (rng.standard_normal(s).astype(np.float32) for s in ((3, 5), (5, 4), (3, 4)))
    dx, dw = cpu.dense_grad(lut, 3, dy, x, w)
    # dX[i][k] = sum_j P(w[k][j], dy[i][j]);  dW[k][j] = sum_i P(x[i][k], dy[i][j])
    assert np.array_equal(dx.view(np.uint32), cpu.gemm(lut, 3, w, dy, transB=True).T.copy().view(np.uint32))
    assert np.array_equal(dw.view(np.uint32), cpu.gemm(lut, 3, x, dy, transA=True).view(np.uint32))


@pytest.mark.parametrize("ba,bb", [(0, 0), (3, 3), (3, 1), (1, 3), (3, 0), (0, 3)])
def test_matmul_shape_cases(ba, bb):
    rng = np.random.default_rng(6)
    a = small_ints(rng, ((ba,) if ba else ()) + (5, 6))
    b = small_ints(rng, ((bb,) if bb else ()) + (6, 4))
    assert np.array_equal(cpu.matmul(ACC7, 7, a, b), np.matmul(a, b))


def test_matmul_rejects_mismatch():
    with pytest.raises(ValueError):
        cpu.matmul(ACC7, 7, np.zeros((2, 3), np.float32), np.zeros((4, 5), np.float32))


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("padding", ["VALID", "SAME"])
@pytest.mark.parametrize("shape", [s for s in REF_CONV_SHAPES if s[0] * s[1] * s[2] <= 4 * 14 * 14 + 400])
def test_conv_equals_library_conv_and_autograd(shape, stride, padding):
    n, h, w_, c, kh, kw, _, oc = shape
    if padding == "VALID" and (kh > h or kw > w_):
        pytest.skip("empty VALID output")
    rng = np.random.default_rng(hash(shape) % 1000 + stride)
    x = small_ints(rng, (n, h, w_, c), -2, 2)  # the reference test's own operand range
    w = small_ints(rng, (kh, kw, c, oc), -2, 2)
    y = cpu.conv2d_fwd(ACC7, 7, x, w, (stride, stride), padding)
    dy = small_ints(rng, y.shape, -2, 2)
    y_ref, dx_ref, dw_ref = torch_conv_reference(x, w, dy, (stride, stride), padding)
    assert y.shape == y_ref.shape
    assert np.array_equal(y.astype(np.float64), y_ref)
    dx = cpu.conv2d_grad_input(ACC7, 7, x.shape, w, dy, (stride, stride), padding)
    dw = cpu.conv2d_grad_filter(ACC7, 7, x, w.shape, dy, (stride, stride), padding)
    assert np.array_equal(dx.astype(np.float64), dx_ref)
    assert np.array_equal(dw.astype(np.float64), dw_ref)


@pytest.mark.parametrize("shape,stride,padding", [((128, 32, 32, 1, 5, 5, 1, 6), 1, "SAME"),
                                                  ((128, 14, 14, 6, 5, 5, 6, 16), 2, "VALID")])
def test_conv_lenet_like_shapes_of_reference_test(shape, stride, padding):
    n, h, w_, c, kh, kw, _, oc = shape
    n = 8  # same geometry, fewer images, to keep the CPU suite short
    rng = np.random.default_rng(11)
    x, w = small_ints(rng, (n, h, w_, c), -2, 2), small_ints(rng, (kh, kw, c, oc), -2, 2)
    y = cpu.conv2d_fwd(ACC7, 7, x, w, (stride, stride), padding)
    dy = small_ints(rng, y.shape, -2, 2)
    y_ref, dx_ref, dw_ref = torch_conv_reference(x, w, dy, (stride, stride), padding)
    assert np.array_equal(y.astype(np.float64), y_ref)
    assert np.array_equal(cpu.conv2d_grad_input(ACC7, 7, x.shape, w, dy, (stride, stride), padding).astype(np.float64), dx_ref)
    assert np.array_equal(cpu.conv2d_grad_filter(ACC7, 7, x, w.shape, dy, (stride, stride), padding).astype(np.float64), dw_ref)


def test_conv_operand_order():
    """fwd P(input, filter); grad-input P(grad, filter); grad-filter P(input, grad)."""
    lut = asym_lut(3)
    rng = np.random.default_rng(12)
    x = rng.standard_normal((1, 1, 1, 1)).astype(np.float32)
    w = rng.standard_normal((1, 1, 1, 1)).astype(np.float32)
    dy = rng.standard_normal((1, 1, 1, 1)).astype(np.float32)
    p = lambda a, b: cpu.lut_mul_array(lut, 3, a.ravel(), b.ravel())[0]
    assert cpu.conv2d_fwd(lut, 3, x, w, (1, 1), "VALID").ravel()[0] == p(x, w)
    assert cpu.conv2d_grad_input(lut, 3, x.shape, w, dy, (1, 1), "VALID").ravel()[0] == p(dy, w)
    assert cpu.conv2d_grad_filter(lut, 3, x, w.shape, dy, (1, 1), "VALID").ravel()[0] == p(x, dy)
    assert p(x, w) != p(w, x)


def test_conv_equals_im2col_gemm_bitwise_with_real_multiplier():
    """The direct loop nest and the reference's lowering (im2col rows in
    (fy, fx, c) order times the HWIO filter matrix) are the same FP32 sum."""
    rng = np.random.default_rng(13)
    x = np.maximum(rng.standard_normal((2, 6, 5, 3)), 0).astype(np.float32)
    w = rng.standard_normal((3, 2, 3, 4)).astype(np.float32)
    y = cpu.conv2d_fwd(MBM7, 7, x, w, (1, 1), "SAME")
    oh, pt = cpu.conv_geometry(6, 3, 1, "SAME")
    ow, pl = cpu.conv_geometry(5, 2, 1, "SAME")
    cols = np.zeros((2 * oh * ow, 3 * 2 * 3), np.float32)
    r = 0
    for b in range(2):
        for oy in range(oh):
            for ox in range(ow):
                for fy in range(3):
                    for fx in range(2):
                        iy, ix = oy - pt + fy, ox - pl + fx
                        if 0 <= iy < 6 and 0 <= ix < 5:
                            cols[r, (fy * 2 + fx) * 3:(fy * 2 + fx) * 3 + 3] = x[b, iy, ix]
                r += 1
    want = cpu.gemm(MBM7, 7, cols, w.reshape(18, 4)).reshape(y.shape)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
