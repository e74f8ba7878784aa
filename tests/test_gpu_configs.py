"""The benchmark configurations at their full sizes, on the GPU through the C
ABI.  Where the CPU oracle finishes in seconds the whole result is compared;
at the large sizes, sampled outputs are recomputed by the oracle and
size-independent properties are checked (additivity of the filter gradient
over the batch, image-wise independence of forward / input gradient).
Tolerance: 1e-5 * sum_k |product| (the task's bar), written below."""
import math

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, dev, host, lut32
from tests.util import lut_path, torch_conv_reference

pytestmark = pytest.mark.gpu
REL = 1e-5


def glorot(rng, shape, fan_in, fan_out):
    lim = math.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-lim, lim, shape).astype(np.float32)


def conv_abs_bounds(x, w, dy, st, padding):
    return torch_conv_reference(np.abs(x), np.abs(w), np.abs(dy), st, padding)


def test_cfg2_lenet5_convs_mitchell7_full_size():
    """LeNet-5: conv1 5x5 1->6 SAME on [256,28,28,1] uniform[0,1); conv2 5x5
    6->16 VALID on [256,14,14,6] half-normal; Glorot-uniform filters;
    upstream gradients N(0, 0.1); MIT_7; forward + both gradients."""
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(lut_path("MIT", 7))
    L = lut32("MIT", 7)
    cases = [
        ((256, 28, 28, 1), (5, 5, 1, 6), "SAME", 3, 4, 7),
        ((256, 14, 14, 6), (5, 5, 6, 16), "VALID", 5, 6, 8),
    ]
    for xs, ws, padding, sx, sw, sg in cases:
        x = np.random.default_rng(sx).random(xs, dtype=np.float32) if xs[3] == 1 else \
            np.abs(np.random.default_rng(sx).standard_normal(xs)).astype(np.float32)
        w = glorot(np.random.default_rng(sw), ws, ws[0] * ws[1] * ws[2], ws[0] * ws[1] * ws[3])
        y_ref = cpu.conv2d_fwd(L, 7, x, w, (1, 1), padding, threads=8)
        dy = (np.random.default_rng(sg).standard_normal(y_ref.shape) * 0.1).astype(np.float32)
        dx_ref = cpu.conv2d_grad_input(L, 7, xs, w, dy, (1, 1), padding, threads=8)
        dw_ref = cpu.conv2d_grad_filter(L, 7, x, ws, dy, (1, 1), padding, threads=8)
        s_y, s_dx, s_dw = conv_abs_bounds(x, w, dy, (1, 1), padding)
        y = host(functors.convam(lut, dev(x), dev(w), (1, 1), padding))
        dx = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), (1, 1), padding))
        dw = host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), (1, 1), padding))
        assert_close_sum_abs(y, y_ref, s_y, REL)
        assert_close_sum_abs(dx, dx_ref, s_dx, REL)
        assert_close_sum_abs(dw, dw_ref, s_dw, REL)


@pytest.fixture(scope="module")
def cfg3():
    xs, ws = (32, 56, 56, 64), (3, 3, 64, 64)
    x = np.maximum(np.random.default_rng(9).standard_normal(xs), 0).astype(np.float32)
    w = (np.random.default_rng(10).standard_normal(ws) * np.sqrt(2.0 / 576)).astype(np.float32)
    dy = np.random.default_rng(11).standard_normal(xs).astype(np.float32)
    return xs, ws, x, w, dy


def test_cfg3_resnet50_3x3_full_size_forward_and_input_grad(cfg3):
    """Full-size launch; the first and last image (which the tail launch
    covers) are recomputed by the oracle."""
    from approxtrain_amd import ApproxMulLut, functors
    xs, ws, x, w, dy = cfg3
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    y = host(functors.convam(lut, dev(x), dev(w), (1, 1), "SAME"))
    dx = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), (1, 1), "SAME"))
    for img in (0, 31):
        xi, dyi = x[img:img + 1], dy[img:img + 1]
        y_ref = cpu.conv2d_fwd(L, 7, xi, w, (1, 1), "SAME", threads=8)
        dx_ref = cpu.conv2d_grad_input(L, 7, xi.shape, w, dyi, (1, 1), "SAME", threads=8)
        s_y, s_dx, _ = conv_abs_bounds(xi, w, dyi, (1, 1), "SAME")
        assert_close_sum_abs(y[img:img + 1], y_ref, s_y, REL)
        assert_close_sum_abs(dx[img:img + 1], dx_ref, s_dx, REL)
    # image-wise independence: a sub-batch gives the same values as the full batch
    y_sub = host(functors.convam(lut, dev(x[8:12]), dev(w), (1, 1), "SAME"))
    s_sub, _, _ = torch_conv_reference(np.abs(x[8:12]), np.abs(w), None, (1, 1), "SAME")
    assert_close_sum_abs(y_sub, y[8:12], s_sub, REL)


def test_cfg3_resnet50_3x3_full_size_filter_grad(cfg3):
    """grad-filter reduces over all 100 352 pixels: check it against the oracle
    on a 2-image slice, and the full batch through additivity over the batch."""
    from approxtrain_amd import ApproxMulLut, functors
    xs, ws, x, w, dy = cfg3
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    dw2 = host(functors.convam_filter_grad(lut, dev(x[:2]), ws, dev(dy[:2]), (1, 1), "SAME"))
    ref2 = cpu.conv2d_grad_filter(L, 7, x[:2], ws, dy[:2], (1, 1), "SAME", threads=8)
    _, _, s2 = conv_abs_bounds(x[:2], w, dy[:2], (1, 1), "SAME")
    assert_close_sum_abs(dw2, ref2, s2, REL)
    full = host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), (1, 1), "SAME")).astype(np.float64)
    parts = sum(host(functors.convam_filter_grad(lut, dev(x[i:i + 8]), ws, dev(dy[i:i + 8]), (1, 1), "SAME")).astype(np.float64)
                for i in range(0, 32, 8))
    _, _, s_full = conv_abs_bounds(x, w, dy, (1, 1), "SAME")
    assert_close_sum_abs(full, parts, s_full, REL)


@pytest.mark.parametrize("kind,m", [(k, m) for k in ("MBM", "MIT") for m in (1, 3, 5, 7, 11)])
def test_cfg4_square_gemm_4096_sampled_against_oracle(kind, m):
    """C = A.B, dA = dC.B^T, dB = A^T.dC at 4096^3 for every table of the sweep: 48 x 48 sampled
    outputs of each are recomputed by the oracle (full-length 4096-term reductions).  The width-11
    tables come from the generator: no reference file or model exists above width 7, so their
    parity is unpinned beyond the closed-form rule that reproduces every reference file; the
    test pins the multiply-accumulate through the table, not the table."""
    from approxtrain_amd import ApproxMulLut, functors
    if m <= 7:
        lut = ApproxMulLut.cached(lut_path(kind, m))
        L = lut32(kind, m)
    else:
        L = cpu.lutgen32(kind, m)
        lut = ApproxMulLut.from_entries((((L >> 23) << 31) | (L & 0x7fffff)).astype(np.uint32), m)
    n = 4096
    A = np.random.default_rng(12).standard_normal((n, n)).astype(np.float32)
    B = np.random.default_rng(13).standard_normal((n, n)).astype(np.float32)
    dC = np.random.default_rng(14).standard_normal((n, n)).astype(np.float32)
    Ad, Bd, dCd = dev(A), dev(B), dev(dC)
    rows = np.random.default_rng(15).choice(n, 48, replace=False)
    cols = np.random.default_rng(16).choice(n, 48, replace=False)
    C = host(functors.gemm(lut, Ad, Bd))[np.ix_(rows, cols)]
    a_s, b_s = A[rows], np.ascontiguousarray(B[:, cols])
    assert_close_sum_abs(C, cpu.gemm(L, m, a_s, b_s), cpu.gemm_abs(L, m, a_s, b_s), REL)
    dA = host(functors.gemm(lut, dCd, Bd, trans_b=True))[np.ix_(rows, cols)]      # P(dC, B)
    g_s, bt_s = dC[rows], B[cols]
    assert_close_sum_abs(dA, cpu.gemm(L, m, g_s, bt_s, transB=True), cpu.gemm_abs(L, m, g_s, bt_s, transB=True), REL)
    dB = host(functors.gemm(lut, Ad, dCd, trans_a=True))[np.ix_(rows, cols)]      # P(A, dC)
    at_s, g2_s = np.ascontiguousarray(A[:, rows]), np.ascontiguousarray(dC[:, cols])
    assert_close_sum_abs(dB, cpu.gemm(L, m, at_s, g2_s, transA=True), cpu.gemm_abs(L, m, at_s, g2_s, transA=True), REL)


def test_cfg5_ammha_block_full_size():
    """Encoder attention block b=32, s=256, d_model=512, 8 heads, MBM_7:
    forward + backward run; the Q projection, one head's QK^T and PV, and the
    weight gradient of the output projection are sampled against the oracle."""
    from approxtrain_amd.layers import MultiHeadAttention
    from approxtrain_amd.math_ops import matmulam
    MBM = lut_path("MBM", 7)
    L = lut32("MBM", 7)
    b, s, d, h = 32, 256, 512, 8
    x = np.random.default_rng(15).standard_normal((b, s, d)).astype(np.float32)
    mha = MultiHeadAttention(MBM, h, d, d, d, input_dim=d).cuda()
    with torch.no_grad():
        for seed, layer in zip((16, 17, 18, 19), (mha.W_q, mha.W_k, mha.W_v, mha.W_o)):
            layer.kernel.copy_(dev(glorot(np.random.default_rng(seed), (d, d), d, d)))
    xd = dev(x).requires_grad_(True)
    y = mha(xd, xd, xd)
    assert tuple(y.shape) == (b, s, d) and torch.isfinite(y).all()
    y.backward(torch.ones_like(y))
    assert torch.isfinite(xd.grad).all() and all(torch.isfinite(p.grad).all() for p in mha.parameters())
    # projection [8192,512].[512,512]: 32 x 32 sampled outputs
    rows = np.random.default_rng(1).choice(b * s, 32, replace=False)
    cols = np.random.default_rng(2).choice(d, 32, replace=False)
    wq = host(mha.W_q.kernel)
    q = host(mha.W_q(xd.detach())).reshape(b * s, d)
    xs_, ws_ = x.reshape(b * s, d)[rows], np.ascontiguousarray(wq[:, cols])
    assert_close_sum_abs(q[np.ix_(rows, cols)], cpu.gemm(L, 7, xs_, ws_), cpu.gemm_abs(L, 7, xs_, ws_), REL)
    # one (batch, head) of QK^T and PV from the strided-batch launches
    qh = mha.reshape_tensor(mha.W_q(xd.detach()), h, True)
    kh = mha.reshape_tensor(mha.W_k(xd.detach()), h, True)
    vh = mha.reshape_tensor(mha.W_v(xd.detach()), h, True)
    sc = matmulam(qh, kh, transpose_b=True, mant_mul_lut=MBM)
    qn, kn = host(qh)[5, 3], host(kh)[5, 3]
    assert_close_sum_abs(host(sc)[5, 3], cpu.gemm(L, 7, qn, kn, transB=True), cpu.gemm_abs(L, 7, qn, kn, transB=True), REL)
    p = torch.softmax(sc / math.sqrt(d), dim=-1)
    o = matmulam(p, vh, mant_mul_lut=MBM)
    pn, vn = host(p)[31, 7], host(vh)[31, 7]
    assert_close_sum_abs(host(o)[31, 7], cpu.gemm(L, 7, pn, vn), cpu.gemm_abs(L, 7, pn, vn), REL)
    # weight gradient of a projection: dW = X^T . dY over 8192 rows (split-K): sampled columns
    from approxtrain_amd import functors
    dyp = np.random.default_rng(3).standard_normal((b * s, d)).astype(np.float32)
    _, dw = functors.denseam_grad(MBM, dev(dyp), dev(x.reshape(b * s, d)), mha.W_q.kernel.detach())
    r2 = np.random.default_rng(4).choice(d, 24, replace=False)
    xt_s, g_s = np.ascontiguousarray(x.reshape(b * s, d)[:, r2]), np.ascontiguousarray(dyp[:, cols])
    assert_close_sum_abs(host(dw)[np.ix_(r2, cols)], cpu.gemm(L, 7, xt_s, g_s, transA=True),
                         cpu.gemm_abs(L, 7, xt_s, g_s, transA=True), REL)
