"""Op / gradient wiring of the Python layer on the GPU: amconvolution_v2,
matmulam, denseam and the attention block, against the CPU oracle and, with
the exact-on-integers ACC_7 table, against torch.autograd."""
import math

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, dev, host, lut32
from tests.util import lut_path, small_ints

pytestmark = pytest.mark.gpu
ACC = lut_path("ACC", 7)
MBM = lut_path("MBM", 7)


@pytest.fixture(autouse=True)
def _unsplit():
    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(0)
    yield
    lib.amsim_set_split_k(1)


@pytest.mark.parametrize("stride,padding", [(1, "SAME"), (2, "SAME"), (1, "VALID"), (2, "VALID")])
def test_amconvolution_autograd_matches_torch_on_integers(stride, padding):
    from approxtrain_amd.amnn_ops import amconvolution_v2
    from tests.util import torch_conv_reference
    rng = np.random.default_rng(1)
    x, w = small_ints(rng, (3, 9, 8, 4), -2, 2), small_ints(rng, (3, 3, 4, 6), -2, 2)
    xt, wt = dev(x).requires_grad_(True), dev(w).requires_grad_(True)
    y = amconvolution_v2(xt, wt, strides=[1, stride, stride, 1], padding=padding, mant_mul_lut=ACC)
    dy = small_ints(rng, tuple(y.shape), -2, 2)
    y.backward(dev(dy))
    y_ref, dx_ref, dw_ref = torch_conv_reference(x, w, dy, (stride, stride), padding)
    assert np.array_equal(host(y).astype(np.float64), y_ref)
    assert np.array_equal(host(xt.grad).astype(np.float64), dx_ref)
    assert np.array_equal(host(wt.grad).astype(np.float64), dw_ref)


def test_amconvolution_gradients_are_the_grad_ops():
    """grad_input = ConvamInputGrad(shape(input), filter, dy); grad_filter =
    ConvamFilterGrad(shape(filter), input, dy)  (amnn_ops.py:231-244)."""
    from approxtrain_amd.amnn_ops import amconvolution_v2
    L = lut32("MBM", 7)
    rng = np.random.default_rng(2)
    xs, ws = (2, 10, 10, 32), (3, 3, 32, 16)
    x = np.maximum(rng.standard_normal(xs), 0).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.1).astype(np.float32)
    xt, wt = dev(x).requires_grad_(True), dev(w).requires_grad_(True)
    y = amconvolution_v2(xt, wt, strides=1, padding="SAME", mant_mul_lut=MBM)
    dy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(dev(dy))
    assert np.array_equal(host(y).view(np.uint32), cpu.conv2d_fwd(L, 7, x, w, (1, 1), "SAME").view(np.uint32))
    assert np.array_equal(host(xt.grad).view(np.uint32),
                          cpu.conv2d_grad_input(L, 7, xs, w, dy, (1, 1), "SAME").view(np.uint32))
    assert np.array_equal(host(wt.grad).view(np.uint32),
                          cpu.conv2d_grad_filter(L, 7, x, ws, dy, (1, 1), "SAME").view(np.uint32))


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmulam_forward_and_gradient_formulas(ta, tb):
    """The four transpose cases of math_ops.py:141-157, each gradient being a
    MatMulAM with (first, second) LUT operand order; checked against the
    oracle GEMM and (ACC_7, integers) against torch.autograd."""
    from approxtrain_amd.math_ops import matmulam
    rng = np.random.default_rng(3)
    M, N, K = 20, 12, 17
    a = small_ints(rng, (K, M) if ta else (M, K))
    b = small_ints(rng, (N, K) if tb else (K, N))
    at, bt = dev(a).requires_grad_(True), dev(b).requires_grad_(True)
    out = matmulam(at, bt, transpose_a=ta, transpose_b=tb, mant_mul_lut=ACC)
    g = small_ints(rng, (M, N))
    out.backward(dev(g))
    a64 = torch.tensor(a, dtype=torch.float64, requires_grad=True)
    b64 = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    ref = torch.matmul(a64.T if ta else a64, b64.T if tb else b64)
    ref.backward(torch.tensor(g, dtype=torch.float64))
    assert np.array_equal(host(out).astype(np.float64), ref.detach().numpy())
    assert np.array_equal(host(at.grad).astype(np.float64), a64.grad.numpy())
    assert np.array_equal(host(bt.grad).astype(np.float64), b64.grad.numpy())
    # real multiplier: forward equals the oracle GEMM bit for bit
    L = lut32("MBM", 7)
    a2, b2 = rng.standard_normal(a.shape).astype(np.float32), rng.standard_normal(b.shape).astype(np.float32)
    got = host(matmulam(dev(a2), dev(b2), transpose_a=ta, transpose_b=tb, mant_mul_lut=MBM))
    assert np.array_equal(got.view(np.uint32), cpu.gemm(L, 7, a2, b2, transA=ta, transB=tb).view(np.uint32))


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmulam_gradient_operand_order_with_asymmetric_lut(ta, tb, tmp_path):
    """The reference's op is handed operands that Python already transposed and never sees the
    flags (math_ops.py:92-93), so its gradients are MatMulAM(grad, b_op^T) and
    MatMulAM(a_op^T, grad) (math_ops.py:145-147): the LUT is fed (grad, b) and (a, grad) in
    every transpose case.  An order-sensitive table makes any other order visible."""
    from approxtrain_amd.math_ops import matmulam
    from tests.gpu_util import asym_lut_u8
    tab = asym_lut_u8(3)
    path = tmp_path / "ASYM_3.bin"
    path.write_bytes(tab.tobytes())
    L = cpu.expand_u8(tab, 3)
    rng = np.random.default_rng(11 + 2 * ta + tb)
    M, N, K = 37, 21, 45
    a = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    g = rng.standard_normal((M, N)).astype(np.float32)
    at, bt = dev(a).requires_grad_(True), dev(b).requires_grad_(True)
    matmulam(at, bt, transpose_a=ta, transpose_b=tb, mant_mul_lut=str(path)).backward(dev(g))
    a_op = np.ascontiguousarray(a.T if ta else a)
    b_op = np.ascontiguousarray(b.T if tb else b)
    ga_op = cpu.gemm(L, 3, g, b_op, transB=True)
    gb_op = cpu.gemm(L, 3, a_op, g, transA=True)
    want_a = np.ascontiguousarray(ga_op.T if ta else ga_op)
    want_b = np.ascontiguousarray(gb_op.T if tb else gb_op)
    assert np.array_equal(host(at.grad).view(np.uint32), want_a.view(np.uint32))
    assert np.array_equal(host(bt.grad).view(np.uint32), want_b.view(np.uint32))
    # and the other order really differs with this table
    assert not np.array_equal(cpu.gemm(L, 3, g, b_op, transB=True, swap=True).view(np.uint32), ga_op.view(np.uint32))


def test_matmulam_rank4_and_broadcast_gradient():
    from approxtrain_amd.math_ops import matmulam
    rng = np.random.default_rng(4)
    q, k = small_ints(rng, (2, 3, 5, 4), -3, 3), small_ints(rng, (2, 3, 6, 4), -3, 3)
    qt, kt = dev(q).requires_grad_(True), dev(k).requires_grad_(True)
    s = matmulam(qt, kt, transpose_b=True, mant_mul_lut=ACC)
    assert tuple(s.shape) == (2, 3, 5, 6)
    g = small_ints(rng, (2, 3, 5, 6), -3, 3)
    s.backward(dev(g))
    q64, k64 = torch.tensor(q, dtype=torch.float64, requires_grad=True), torch.tensor(k, dtype=torch.float64, requires_grad=True)
    ref = q64 @ k64.transpose(-1, -2)
    ref.backward(torch.tensor(g, dtype=torch.float64))
    assert np.array_equal(host(s).astype(np.float64), ref.detach().numpy())
    assert np.array_equal(host(qt.grad).astype(np.float64), q64.grad.numpy())
    assert np.array_equal(host(kt.grad).astype(np.float64), k64.grad.numpy())
    # rank-3 x rank-2: the shared operand's gradient sums over the batch
    a, w = small_ints(rng, (4, 5, 6), -3, 3), small_ints(rng, (6, 7), -3, 3)
    at, wt = dev(a).requires_grad_(True), dev(w).requires_grad_(True)
    out = matmulam(at, wt, mant_mul_lut=ACC)
    g = small_ints(rng, (4, 5, 7), -3, 3)
    out.backward(dev(g))
    assert np.array_equal(host(wt.grad).astype(np.float64), np.einsum("bij,bik->jk", a.astype(np.float64), g.astype(np.float64)))


def test_denseam_layer_forward_backward():
    from approxtrain_amd.layers import denseam
    rng = np.random.default_rng(5)
    layer = denseam(10, activation=torch.relu, mant_mul_lut=ACC, input_dim=16).cuda()
    w, b = small_ints(rng, (16, 10), -2, 2), small_ints(rng, (10,), -2, 2)
    with torch.no_grad():
        layer.kernel.copy_(dev(w)); layer.bias.copy_(dev(b))
    x = small_ints(rng, (7, 16), -2, 2)
    xt = dev(x).requires_grad_(True)
    y = layer(xt)
    g = small_ints(rng, (7, 10), -2, 2)
    y.backward(dev(g))
    x64 = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    w64 = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    ref = torch.relu(x64 @ w64 + torch.tensor(b, dtype=torch.float64))
    ref.backward(torch.tensor(g, dtype=torch.float64))
    assert np.array_equal(host(y).astype(np.float64), ref.detach().numpy())
    assert np.array_equal(host(xt.grad).astype(np.float64), x64.grad.numpy())
    assert np.array_equal(host(layer.kernel.grad).astype(np.float64), w64.grad.numpy())
    # rank-3 inputs go through the approximate op too
    y3 = layer(dev(small_ints(rng, (2, 3, 16), -2, 2)))
    assert tuple(y3.shape) == (2, 3, 10)


def test_amconv2d_layer_matches_functor():
    from approxtrain_amd import functors
    from approxtrain_amd.layers import AMConv2D
    torch.manual_seed(0)
    layer = AMConv2D(6, 5, padding="same", mant_mul_lut=MBM, in_channels=1).cuda()
    x = torch.rand(4, 28, 28, 1, device="cuda")
    y = layer(x)
    want = functors.convam(MBM, x, layer.kernel.detach(), (1, 1), "SAME") + layer.bias.detach()
    assert torch.equal(y, want)


def test_multihead_attention_block_against_oracle_composition():
    """AMMHA forward at a small size: the four projections and both attention
    products must equal the same composition built from oracle GEMMs."""
    from approxtrain_amd.layers import MultiHeadAttention
    L = lut32("MBM", 7)
    torch.manual_seed(1)
    b, s, d, h = 2, 16, 32, 4
    mha = MultiHeadAttention(MBM, h, d, d, d, input_dim=d).cuda()
    x = torch.randn(b, s, d, device="cuda")
    y = mha(x, x, x)
    assert tuple(y.shape) == (b, s, d)
    xn = host(x).reshape(b * s, d)

    def proj(layer, inp):
        return cpu.gemm(L, 7, inp, host(layer.kernel)) + host(layer.bias)

    def heads(t):
        return t.reshape(b, s, h, d // h).transpose(0, 2, 1, 3).reshape(b * h, s, d // h)

    q, k, v = heads(proj(mha.W_q, xn)), heads(proj(mha.W_k, xn)), heads(proj(mha.W_v, xn))
    o = np.zeros_like(q)
    for i in range(b * h):
        sc = cpu.gemm(L, 7, q[i], k[i], transB=True) / np.float32(math.sqrt(d))
        wts = torch.softmax(torch.from_numpy(sc), dim=-1).numpy()
        o[i] = cpu.gemm(L, 7, wts, v[i])
    o = o.reshape(b, h, s, d // h).transpose(0, 2, 1, 3).reshape(b * s, d)
    want = proj(mha.W_o, o).reshape(b, s, d)
    np.testing.assert_allclose(host(y), want, rtol=2e-5, atol=2e-6)
    # and it is differentiable end to end
    y.sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in mha.parameters())


def _same_values(a, b):
    """Equal element by element, NaN matching NaN (the sign of a zero is not compared)."""
    a, b = host(a), host(b)
    nan = np.isnan(a)
    return np.array_equal(nan, np.isnan(b)) and np.array_equal(a[~nan], b[~nan])


@pytest.mark.parametrize("split", [0, 1])
@pytest.mark.parametrize("shape,filt,stride,padding", [((3, 9, 11, 8), (3, 3, 8, 20), 1, "SAME"),
                                                        ((2, 12, 12, 4), (5, 5, 4, 3), 2, "VALID"),
                                                        ((40, 14, 14, 32), (3, 3, 32, 64), 1, "SAME")])
def test_fused_bias_relu_epilogue_equals_separate_ops(split, shape, filt, stride, padding):
    """act(conv + bias) computed in the kernel's store (and in the split reduction when the
    reduction is split) holds the same values as the three separate ops."""
    import approxtrain_amd
    from approxtrain_amd import functors
    approxtrain_amd.load_library().amsim_set_split_k(split)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(*shape, device="cuda", generator=g)
    w = torch.randn(*filt, device="cuda", generator=g)
    b = torch.randn(filt[3], device="cuda", generator=g)
    x[0, 1, 2, 0] = float("nan")
    plain = functors.convam(MBM, x, w, (stride, stride), padding)
    assert _same_values(functors.convam(MBM, x, w, (stride, stride), padding, bias=b), plain + b)
    assert _same_values(functors.convam(MBM, x, w, (stride, stride), padding, activation="relu"), torch.relu(plain))
    assert _same_values(functors.convam(MBM, x, w, (stride, stride), padding, bias=b, activation="relu"),
                        torch.relu(plain + b))


@pytest.mark.parametrize("batch,units,width", [(7, 10, 16), (300, 5, 64), (5, 300, 64), (128, 300, 784)])
def test_fused_dense_epilogue_both_orientations(batch, units, width):
    """The bias runs along the output's columns whichever GEMM dimension the kernel spreads over its lanes."""
    from approxtrain_amd import functors
    g = torch.Generator(device="cuda").manual_seed(4)
    x, w, b = (torch.randn(batch, width, device="cuda", generator=g), torch.randn(width, units, device="cuda", generator=g),
               torch.randn(units, device="cuda", generator=g))
    plain = functors.denseam(MBM, x, w)
    assert _same_values(functors.denseam(MBM, x, w, bias=b, activation="relu"), torch.relu(plain + b))
    assert _same_values(functors.denseam(MBM, x, w, bias=b), plain + b)


def test_fused_epilogue_argument_errors():
    from approxtrain_amd import functors
    x, w = torch.zeros(1, 4, 4, 2, device="cuda"), torch.zeros(3, 3, 2, 5, device="cuda")
    with pytest.raises(ValueError):
        functors.convam(MBM, x, w, bias=torch.zeros(4, device="cuda"))
    with pytest.raises(ValueError):
        functors.convam(MBM, x, w, activation="tanh")


def test_amconv2d_layer_fused_gradients_match_torch_on_integers():
    """AMConv2D with bias and ReLU (one fused forward kernel): output, input / kernel / bias gradients
    against float64 torch autograd, exact on small integers with the ACC_7 table."""
    from approxtrain_amd.layers import AMConv2D
    rng = np.random.default_rng(8)
    layer = AMConv2D(5, 3, strides=(2, 2), padding="same", activation="relu", mant_mul_lut=ACC, in_channels=4).cuda()
    w, b = small_ints(rng, (3, 3, 4, 5), -2, 2), small_ints(rng, (5,), -2, 2)
    with torch.no_grad():
        layer.kernel.copy_(dev(w)); layer.bias.copy_(dev(b))
    x = small_ints(rng, (2, 9, 7, 4), -2, 2)
    xt = dev(x).requires_grad_(True)
    y = layer(xt)
    gy = small_ints(rng, tuple(y.shape), -2, 2)
    y.backward(dev(gy))
    x64 = torch.tensor(x, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    w64 = torch.tensor(w, dtype=torch.float64).permute(3, 2, 0, 1).requires_grad_(True)
    b64 = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    # SAME with stride 2 on 9 x 7: output 5 x 4, total padding (2, 2) -> 1 before, 1 after
    ref = torch.relu(torch.nn.functional.conv2d(torch.nn.functional.pad(x64, (1, 1, 1, 1)), w64, b64, stride=2))
    ref.backward(torch.tensor(gy, dtype=torch.float64).permute(0, 3, 1, 2))
    assert np.array_equal(host(y).astype(np.float64), ref.detach().permute(0, 2, 3, 1).numpy())
    assert np.array_equal(host(xt.grad).astype(np.float64), x64.grad.permute(0, 2, 3, 1).numpy())
    assert np.array_equal(host(layer.kernel.grad).astype(np.float64), w64.grad.permute(2, 3, 1, 0).numpy())
    assert np.array_equal(host(layer.bias.grad).astype(np.float64), b64.grad.numpy())
