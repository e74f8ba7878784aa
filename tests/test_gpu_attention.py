"""Dot-product attention through the C ABI (amsim_attention_f32 and its gradient):
both matrix products against the oracle GEMM, bit for bit, evaluated on the
intermediates the library itself produced; the FP32 row steps (division, mask,
softmax and its gradient) against numpy -- the softmax within a few ulps (the
device's expf is not numpy's), its gradient bit for bit by following the
kernel's summation order."""
import math

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import asym_lut_u8, dev, host, lut32
from tests.util import lut_path

pytestmark = pytest.mark.gpu
MBM = lut_path("MBM", 7)


@pytest.fixture(autouse=True)
def _unsplit():
    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(0)
    yield
    lib.amsim_set_split_k(1)


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _softmax64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def _wave_sum(per_lane):
    """Sum over 64 lanes in the order of a xor-butterfly (32, 16, ..., 1), FP32."""
    v = per_lane.astype(np.float32).copy()
    lanes = np.arange(64)
    for o in (32, 16, 8, 4, 2, 1):
        v = (v + v[..., lanes ^ o]).astype(np.float32)
    return v[..., 0]


def _softmax_grad_like_the_kernel(w, g, divisor):
    """d(scores) = (g - sum_j g_j w_j) * w / divisor in the kernel's order of additions.  Rows
    of up to 1024 columns, a multiple of four: lane l adds columns 4l .. 4l+3, then the same
    256 further on, ...; other rows: lane l adds columns l, l + 64, ...; the 64 lanes are then
    combined by a butterfly.  (Slots past the end of a row add +0, which changes nothing.)"""
    cols = w.shape[-1]
    vec = cols % 4 == 0 and cols <= 1024
    group = 256 if vec else 64
    pad = (-cols) % group
    gp = np.pad(g, [(0, 0)] * (g.ndim - 1) + [(0, pad)]).astype(np.float32)
    wp = np.pad(w, [(0, 0)] * (w.ndim - 1) + [(0, pad)]).astype(np.float32)
    prod = (gp * wp).astype(np.float32)
    acc = np.zeros(g.shape[:-1] + (64,), np.float32)
    if vec:
        prod = prod.reshape(g.shape[:-1] + (-1, 64, 4))           # [.., i, lane, component]
        for i in range(prod.shape[-3]):
            for e in range(4):
                acc = (acc + prod[..., i, :, e]).astype(np.float32)
    else:
        prod = prod.reshape(g.shape[:-1] + (-1, 64))              # [.., i, lane]
        for i in range(prod.shape[-2]):
            acc = (acc + prod[..., i, :]).astype(np.float32)
    dot = _wave_sum(acc)[..., None]
    return (((g - dot).astype(np.float32) * w).astype(np.float32) / np.float32(divisor)).astype(np.float32)


@pytest.mark.parametrize("lead,sq,sk,dk,dv,masked", [
    ((3,), 40, 56, 24, 16, False),
    ((2, 4), 64, 64, 32, 32, True),
    ((5,), 7, 130, 9, 3, True),
    ((2,), 20, 600, 8, 8, True),         # three float4 per lane of four
    ((2,), 9, 75, 8, 8, False),          # scalar register path
    ((1,), 33, 1100, 16, 8, False),      # rows longer than the register cache
])
def test_attention_forward_and_gradient(lead, sq, sk, dk, dv, masked):
    from approxtrain_amd import functors
    rng = np.random.default_rng(sq * 7 + sk)
    L = lut32("MBM", 7)
    q = rng.standard_normal(lead + (sq, dk)).astype(np.float32)
    k = rng.standard_normal(lead + (sk, dk)).astype(np.float32)
    v = rng.standard_normal(lead + (sk, dv)).astype(np.float32)
    go = rng.standard_normal(lead + (sq, dv)).astype(np.float32)
    mask = None
    if masked:  # padding mask shared by the heads and by the queries, as an encoder passes it
        mask = (rng.random((lead[0],) + (1,) * (len(lead) - 1) + (1, sk)) < 0.25).astype(np.float32)
    divisor = math.sqrt(float(dk))
    out, w = functors.attention(MBM, dev(q), dev(k), dev(v), divisor, None if mask is None else dev(mask))
    gq, gk, gv = functors.attention_grad(MBM, dev(q), dev(k), dev(v), w, dev(go), divisor)
    out, w, gq, gk, gv = (host(t) for t in (out, w, gq, gk, gv))
    flat = lambda a: a.reshape((-1,) + a.shape[-2:])
    qf, kf, vf, gof, wf, of, gqf, gkf, gvf = map(flat, (q, k, v, go, w, out, gq, gk, gv))
    mf = None if mask is None else flat(np.broadcast_to(mask, lead + (sq, sk)))
    for b in range(qf.shape[0]):
        s = cpu.gemm(L, 7, qf[b], kf[b], transB=True)
        x = (s / np.float32(divisor)).astype(np.float32)
        if mf is not None:
            x = (x + (np.float32(-1e9) * mf[b]).astype(np.float32)).astype(np.float32)
        np.testing.assert_allclose(wf[b], _softmax64(x), rtol=2e-6, atol=1e-30)
        assert np.array_equal(_bits(of[b]), _bits(cpu.gemm(L, 7, wf[b], vf[b]))), f"out, item {b}"
        assert np.array_equal(_bits(gvf[b]), _bits(cpu.gemm(L, 7, wf[b], gof[b], transA=True))), f"d(v), item {b}"
        gw = cpu.gemm(L, 7, gof[b], vf[b], transB=True)
        gs = _softmax_grad_like_the_kernel(wf[b], gw, divisor)
        assert np.array_equal(_bits(gqf[b]), _bits(cpu.gemm(L, 7, gs, kf[b]))), f"d(q), item {b}"
        # d(k) = (q^T . d(scores))^T, the LUT fed as (q, d(scores))
        want_gk = np.ascontiguousarray(cpu.gemm(L, 7, qf[b], gs, transA=True).T)
        assert np.array_equal(_bits(gkf[b]), _bits(want_gk)), f"d(k), item {b}"


def test_attention_operand_order_with_asymmetric_lut():
    """(q, k), (weights, v) forward; (d(out), v), (weights, d(out)), (d(scores), k), (q, d(scores)) backward."""
    from approxtrain_amd import ApproxMulLut, functors
    tab = asym_lut_u8(3)
    lut = ApproxMulLut.from_entries(tab, 3)
    L = cpu.expand_u8(tab, 3)
    rng = np.random.default_rng(5)
    sq, sk, dk, dv = 24, 40, 16, 8
    q, k, v, go = (rng.standard_normal(s).astype(np.float32) for s in ((2, sq, dk), (2, sk, dk), (2, sk, dv), (2, sq, dv)))
    out, w = functors.attention(lut, dev(q), dev(k), dev(v), 4.0)
    gq, gk, gv = functors.attention_grad(lut, dev(q), dev(k), dev(v), w, dev(go), 4.0)
    out, w, gq, gk, gv = (host(t) for t in (out, w, gq, gk, gv))
    for b in range(2):
        x = (cpu.gemm(L, 3, q[b], k[b], transB=True) / np.float32(4.0)).astype(np.float32)
        np.testing.assert_allclose(w[b], _softmax64(x), rtol=2e-6)
        assert np.array_equal(_bits(out[b]), _bits(cpu.gemm(L, 3, w[b], v[b])))
        assert np.array_equal(_bits(gv[b]), _bits(cpu.gemm(L, 3, w[b], go[b], transA=True)))
        gs = _softmax_grad_like_the_kernel(w[b], cpu.gemm(L, 3, go[b], v[b], transB=True), 4.0)
        assert np.array_equal(_bits(gq[b]), _bits(cpu.gemm(L, 3, gs, k[b])))
        assert np.array_equal(_bits(gk[b]), _bits(np.ascontiguousarray(cpu.gemm(L, 3, q[b], gs, transA=True).T)))


def test_attention_core_of_the_encoder_block_at_full_size():
    """The attention core of the benchmark's encoder block -- 32 sequences x 8 heads of 256 positions,
    64 features per head, MBM_7 -- in one library call per direction: for a sample of (sequence, head)
    items both forward products and all four backward products against the oracle GEMM, bit for bit,
    on the intermediates the library produced; every other item must at least be finite."""
    from approxtrain_amd import functors
    rng = np.random.default_rng(77)
    L = lut32("MBM", 7)
    b, h, s, d = 32, 8, 256, 64
    q, k, v, go = (rng.standard_normal((b, h, s, d)).astype(np.float32) for _ in range(4))
    divisor = math.sqrt(float(d))
    out, w = functors.attention(MBM, dev(q), dev(k), dev(v), divisor)
    gq, gk, gv = functors.attention_grad(MBM, dev(q), dev(k), dev(v), w, dev(go), divisor)
    for t in (out, w, gq, gk, gv):
        assert torch.isfinite(t).all()
    out, w, gq, gk, gv = (host(t) for t in (out, w, gq, gk, gv))
    for (i, j) in ((0, 0), (13, 5), (31, 7), (20, 2)):
        x = (cpu.gemm(L, 7, q[i, j], k[i, j], transB=True) / np.float32(divisor)).astype(np.float32)
        np.testing.assert_allclose(w[i, j], _softmax64(x), rtol=2e-6, atol=1e-30)
        assert np.array_equal(_bits(out[i, j]), _bits(cpu.gemm(L, 7, w[i, j], v[i, j]))), f"out, item {i, j}"
        assert np.array_equal(_bits(gv[i, j]), _bits(cpu.gemm(L, 7, w[i, j], go[i, j], transA=True))), f"d(v), item {i, j}"
        gs = _softmax_grad_like_the_kernel(w[i, j], cpu.gemm(L, 7, go[i, j], v[i, j], transB=True), divisor)
        assert np.array_equal(_bits(gq[i, j]), _bits(cpu.gemm(L, 7, gs, k[i, j]))), f"d(q), item {i, j}"
        want_gk = np.ascontiguousarray(cpu.gemm(L, 7, q[i, j], gs, transA=True).T)
        assert np.array_equal(_bits(gk[i, j]), _bits(want_gk)), f"d(k), item {i, j}"


@pytest.mark.parametrize("mask_shape", [None, (2, 1, 1, 48), (48, 48), (2, 1, 48, 48), (2, 3, 48, 48), (1, 3, 1, 48)])
def test_attention_layer_matches_the_composed_ops(mask_shape):
    """DotProductAttention (one library call per direction) against the same chain spelled with
    matmulam and torch ops: identical scores, so weights agree to FP32 rounding; outputs and
    gradients agree up to the few products whose truncated operand differs by one ulp."""
    from approxtrain_amd.layers import DotProductAttention
    from approxtrain_amd.math_ops import matmulam
    rng = np.random.default_rng(9)
    b, h, s, d = 2, 3, 48, 16
    mk = lambda: dev(rng.standard_normal((b, h, s, d)).astype(np.float32)).requires_grad_(True)
    q, k, v = mk(), mk(), mk()
    mask = None if mask_shape is None else dev((rng.random(mask_shape) < 0.3).astype(np.float32))
    go = dev(rng.standard_normal((b, h, s, d)).astype(np.float32))
    DotProductAttention(MBM)(q, k, v, d, mask).backward(go)
    fused = [host(t.grad) for t in (q, k, v)]
    for t in (q, k, v):
        t.grad = None
    sc = matmulam(q, k, transpose_b=True, mant_mul_lut=MBM) / math.sqrt(float(d))
    if mask is not None:
        sc = sc + -1e9 * mask
    matmulam(torch.softmax(sc, dim=-1), v, mant_mul_lut=MBM).backward(go)
    for got, t in zip(fused, (q, k, v)):
        want = host(t.grad)
        assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max()
        assert np.mean(np.abs(got - want) <= 1e-5 * np.abs(want).max()) > 0.98


def test_attention_argument_errors():
    import ctypes as C
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut.cached(MBM)
    z = lambda *s: torch.zeros(*s, device="cuda")
    with pytest.raises(ValueError):
        functors.attention(lut, z(2, 8, 4), z(3, 8, 4), z(3, 8, 4), 2.0)
    with pytest.raises(ValueError):
        functors.attention(lut, z(2, 8, 4), z(2, 8, 5), z(2, 8, 4), 2.0)
    with pytest.raises(ValueError):
        functors.attention(lut, z(2, 8, 4), z(2, 8, 4), z(2, 8, 4), 2.0, mask=z(2, 7, 8))
    with pytest.raises(RuntimeError):
        functors.attention(lut, z(2, 8, 4), z(2, 8, 4), z(2, 8, 4), 0.0)
    # gradient with a workspace one byte short
    n = lib.amsim_attention_grad_workspace_bytes(2, 8, 8, 4, 4)
    ws = torch.empty(n + 256, dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    base = C.c_void_p(ws.data_ptr() + (-ws.data_ptr()) % 256)
    t = z(2, 8, 4)
    w = z(2, 8, 8)
    rc = lib.amsim_attention_grad_f32(lut.handle, p(t), p(t), p(t), p(w), p(t), 2, 8, 8, 4, 4, 2.0, p(z(2, 8, 4)),
                                      p(z(2, 8, 4)), p(z(2, 8, 4)), base, n - 1, None)
    assert rc != 0 and b"workspace" in lib.amsim_last_error()
    # empty batch is a no-op
    out, wts = functors.attention(lut, z(0, 8, 4), z(0, 8, 4), z(0, 8, 4), 2.0)
    assert out.shape == (0, 8, 4) and wts.shape == (0, 8, 8)
