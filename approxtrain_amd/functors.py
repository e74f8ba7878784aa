"""Functor-level calls: one function per device functor of the reference
(convam.h:69-143, denseam.h:7-53, matmulam.h:10-28, cuda/gemm.cu:17), same
argument meaning, operating on CUDA/HIP torch tensors.  torch supplies device
memory, the workspace and the current stream; all arithmetic happens in
libamsim.so."""
import ctypes as C

import torch

from ._lib import check, conv_geometry, load_library
from .lut import ApproxMulLut


def _dev(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a tensor in device memory (there is no CPU path)")
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    return t.contiguous()


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _workspace(nbytes, device):
    if nbytes == 0:
        return None, C.c_void_p(0)
    ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
    off = (-ws.data_ptr()) % 256
    return ws, C.c_void_p(ws.data_ptr() + off)


def _lut(lut):
    if isinstance(lut, ApproxMulLut):
        return lut
    return ApproxMulLut.cached(lut)


def mul(lut, a, b):
    """Elementwise approximate product (test hook)."""
    a, b = _dev(a, "a"), _dev(b, "b")
    lut = _lut(lut)
    if a.shape != b.shape:
        raise ValueError("shape mismatch")
    out = torch.empty_like(a)
    check(load_library().amsim_mul_f32(lut.handle, _ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()))
    return out


def gemm(lut, A, B, trans_a=False, trans_b=False, swap_operands=False):
    """C = op(A) . op(B) for rank-2 A, B, or a strided batch for rank-3
    operands (a rank-2 operand is shared by every batch item)."""
    A, B = _dev(A, "A"), _dev(B, "B")
    lut = _lut(lut)
    if A.dim() not in (2, 3) or B.dim() not in (2, 3):
        raise ValueError("operands must be rank 2 or 3")
    batch = max(A.shape[0] if A.dim() == 3 else 1, B.shape[0] if B.dim() == 3 else 1)
    ra, ca = A.shape[-2:]
    rb, cb = B.shape[-2:]
    M, K = (ca, ra) if trans_a else (ra, ca)
    K2, N = (cb, rb) if trans_b else (rb, cb)
    if K != K2:
        raise ValueError("inner dimensions differ")
    for t in (A, B):
        if t.dim() == 3 and t.shape[0] not in (1, batch):
            raise ValueError("batch sizes differ")
    sA = ra * ca if (A.dim() == 3 and A.shape[0] == batch and batch > 1) else 0
    sB = rb * cb if (B.dim() == 3 and B.shape[0] == batch and batch > 1) else 0
    batched = A.dim() == 3 or B.dim() == 3
    out = torch.empty((batch, M, N) if batched else (M, N), dtype=torch.float32, device=A.device)
    lib = load_library()
    nbytes = lib.amsim_gemm_workspace_bytes_for(lut.handle, int(trans_a), int(trans_b), M, N, K, batch)
    ws, wsp = _workspace(nbytes, A.device)
    check(lib.amsim_gemm_f32(lut.handle, int(trans_a), int(trans_b), int(swap_operands), M, N, K, _ptr(A), ca,
                             _ptr(B), cb, _ptr(out), N, batch, sA, sB, M * N, wsp, nbytes, _stream()))
    return out


ACTIVATIONS = {None: 0, "linear": 0, "relu": 1}


def _epilogue(bias, activation, channels, device):
    """Validates the optional fused epilogue; returns (bias tensor or None, bias pointer, activation code)."""
    if activation not in ACTIVATIONS:
        raise ValueError("fused activation must be None, 'linear' or 'relu'")
    b = None
    if bias is not None:
        b = _dev(bias, "bias")
        if b.dim() != 1 or b.shape[0] != channels:
            raise ValueError("bias must have one entry per output channel")
    return b, (_ptr(b) if b is not None else None), ACTIVATIONS[activation]


def convam(lut, input, filter, strides=(1, 1), padding="SAME", bias=None, activation=None):
    """ConvamFunctor: NHWC input, HWIO filter -> NHWC output.  With ``bias`` / ``activation``
    the layer's BiasAdd and ReLU are applied as the result is stored (same values as the
    separate ops)."""
    x, w = _dev(input, "input"), _dev(filter, "filter")
    b, bptr, act = _epilogue(bias, activation, w.shape[3], x.device)
    lut = _lut(lut)
    n, h, wd, c = x.shape
    kh, kw, c2, oc = w.shape
    if c != c2:
        raise ValueError("input depth must equal filter depth")
    oh, pt = conv_geometry(h, kh, strides[0], padding)
    ow, pl = conv_geometry(wd, kw, strides[1], padding)
    out = torch.empty((n, oh, ow, oc), dtype=torch.float32, device=x.device)
    lib = load_library()
    nbytes = lib.amsim_convam_workspace_bytes_for(lut.handle, n, oh, ow, oc, kh, kw, c)
    ws, wsp = _workspace(nbytes, x.device)
    if b is None and act == 0:
        check(lib.amsim_convam_f32(lut.handle, _ptr(x), _ptr(out), n, oh, ow, oc, strides[1], strides[0], pl, pt,
                                   kh, kw, c, wd, h, _ptr(w), wsp, nbytes, _stream()))
    else:
        check(lib.amsim_convam_bias_act_f32(lut.handle, _ptr(x), _ptr(out), n, oh, ow, oc, strides[1], strides[0],
                                            pl, pt, kh, kw, c, wd, h, _ptr(w), bptr, act, wsp, nbytes, _stream()))
    return out


def convam_input_grad(lut, input_sizes, filter, out_backprop, strides=(1, 1), padding="SAME"):
    """ConvamInputGradFunctor: gradient w.r.t. the NHWC input of shape input_sizes."""
    w, dy = _dev(filter, "filter"), _dev(out_backprop, "out_backprop")
    lut = _lut(lut)
    n, h, wd, c = [int(v) for v in input_sizes]
    kh, kw, c2, oc = w.shape
    oh, pt = conv_geometry(h, kh, strides[0], padding)
    ow, pl = conv_geometry(wd, kw, strides[1], padding)
    if c != c2 or tuple(dy.shape) != (n, oh, ow, oc):
        raise ValueError("out_backprop / filter do not match input_sizes")
    out = torch.empty((n, h, wd, c), dtype=torch.float32, device=dy.device)
    hole_h = (oh - 1) * strides[0] + 1 if oh > 0 else 0
    hole_w = (ow - 1) * strides[1] + 1 if ow > 0 else 0
    lib = load_library()
    nbytes = lib.amsim_convam_input_grad_workspace_bytes_for(lut.handle, n, h, wd, c, kh, kw, oc, strides[0], strides[1],
                                                             kh - 1 - pt, kw - 1 - pl)
    ws, wsp = _workspace(nbytes, dy.device)
    check(lib.amsim_convam_input_grad_f32(lut.handle, _ptr(dy), hole_w, hole_h, kh - 1 - pt, kw - 1 - pl, _ptr(w),
                                          kh, kw, oc, strides[0], strides[1], n, h, wd, c, _ptr(out), oh, ow,
                                          wsp, nbytes, _stream()))
    return out


def convam_filter_grad(lut, input, filter_sizes, out_backprop, strides=(1, 1), padding="SAME"):
    """ConvamFilterGradFunctor: gradient w.r.t. the HWIO filter of shape filter_sizes."""
    x, dy = _dev(input, "input"), _dev(out_backprop, "out_backprop")
    lut = _lut(lut)
    n, h, wd, c = x.shape
    kh, kw, c2, oc = [int(v) for v in filter_sizes]
    oh, pt = conv_geometry(h, kh, strides[0], padding)
    ow, pl = conv_geometry(wd, kw, strides[1], padding)
    if c != c2 or tuple(dy.shape) != (n, oh, ow, oc):
        raise ValueError("out_backprop / input do not match filter_sizes")
    out = torch.empty((kh, kw, c, oc), dtype=torch.float32, device=x.device)
    lib = load_library()
    nbytes = lib.amsim_convam_filter_grad_workspace_bytes_for(lut.handle, n, oh, ow, oc, kh, kw, c)
    ws, wsp = _workspace(nbytes, x.device)
    check(lib.amsim_convam_filter_grad_f32(lut.handle, _ptr(x), _ptr(dy), h, wd, n, c, ow, oh, oc, pl, pt,
                                           strides[0], strides[1], kw, kh, _ptr(out), wsp, nbytes, _stream()))
    return out


def _dense_dims(x, w):
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[0]:
        raise ValueError("denseam expects input [batch, width] and weights [width, units]")
    return x.shape[0], w.shape[1], x.shape[1]


def denseam(lut, inputs, weights, bias=None, activation=None):
    """DenseamFunctor; ``bias`` / ``activation`` fuse the layer's bias_add and ReLU into the store."""
    x, w = _dev(inputs, "inputs"), _dev(weights, "weights")
    batch, units, width = _dense_dims(x, w)
    b, bptr, act = _epilogue(bias, activation, units, x.device)
    lut = _lut(lut)
    out = torch.empty((batch, units), dtype=torch.float32, device=x.device)
    lib = load_library()
    nbytes = lib.amsim_denseam_workspace_bytes_for(lut.handle, batch, units, width)
    ws, wsp = _workspace(nbytes, x.device)
    if b is None and act == 0:
        check(lib.amsim_denseam_f32(lut.handle, _ptr(x), _ptr(w), _ptr(out), batch, units, width, wsp, nbytes,
                                    _stream()))
    else:
        check(lib.amsim_denseam_bias_act_f32(lut.handle, _ptr(x), _ptr(w), _ptr(out), batch, units, width, bptr, act,
                                             wsp, nbytes, _stream()))
    return out


def denseam_grad(lut, grad, inputs, weights):
    """DenseamGrad op: returns (grad_input, grad_weights)."""
    x, w, dy = _dev(inputs, "inputs"), _dev(weights, "weights"), _dev(grad, "grad")
    lut = _lut(lut)
    batch, units, width = _dense_dims(x, w)
    if tuple(dy.shape) != (batch, units):
        raise ValueError("grad must be [batch, units]")
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    lib = load_library()
    nbytes = lib.amsim_denseam_workspace_bytes_for(lut.handle, batch, units, width)
    ws, wsp = _workspace(nbytes, x.device)
    check(lib.amsim_denseam_weight_grad_f32(lut.handle, _ptr(x), _ptr(dy), _ptr(dw), batch, units, width, wsp,
                                            nbytes, _stream()))
    check(lib.amsim_denseam_input_grad_f32(lut.handle, _ptr(w), _ptr(dy), _ptr(dx), batch, units, width, wsp,
                                           nbytes, _stream()))
    return dx, dw


def matmulam(lut, a, b):
    """LaunchMatMul: rank-2 / rank-3 operands with the reference's batch rules."""
    a, b = _dev(a, "a"), _dev(b, "b")
    lut = _lut(lut)
    if a.dim() not in (2, 3) or b.dim() not in (2, 3):
        raise ValueError("Input a and b should be 2 dimensional or 3 dimensional and compitable batch size")
    ba = a.shape[0] if a.dim() == 3 else 0
    bb = b.shape[0] if b.dim() == 3 else 0
    ra, ca = a.shape[-2:]
    rb, cb = b.shape[-2:]
    nb = max(ba, bb)
    out = torch.empty((nb, ra, cb) if (a.dim() == 3 or b.dim() == 3) else (ra, cb), dtype=torch.float32,
                      device=a.device)
    lib = load_library()
    nbytes = lib.amsim_matmulam_workspace_bytes_for(lut.handle, ba, bb, ra, ca, rb, cb)
    ws, wsp = _workspace(nbytes, a.device)
    check(lib.amsim_matmulam_f32(lut.handle, _ptr(a), _ptr(b), ba, bb, ra, ca, rb, cb, _ptr(out), wsp, nbytes,
                                 _stream()))
    if out.numel() and ca == 0:
        pass  # an empty reduction yields zeros (matmulam.cc:154-160); the library writes them
    return out


def _mask_layout(mask, lead, seq_q, seq_k, device):
    """Layout of an attention mask broadcastable to ``lead + (seq_q, seq_k)`` for the library:
    (tensor kept alive, pointer, batch divisor, batch stride, row stride).  A mask shared by the
    trailing leading dimensions (the heads) and / or by the queries is passed as it is; any
    other broadcast pattern is materialised."""
    if mask is None:
        return None, C.c_void_p(0), 1, 0, 0
    m = mask.to(device=device, dtype=torch.float32)
    full = tuple(lead) + (seq_q, seq_k)
    m = m.reshape((1,) * (len(full) - m.dim()) + tuple(m.shape)) if m.dim() < len(full) else m
    if m.dim() != len(full) or any(a not in (1, b) for a, b in zip(m.shape, full)):
        raise ValueError("mask does not broadcast against the attention scores")
    batch = 1
    for d in lead:
        batch *= d
    rows_shared = m.shape[-2] == 1 and seq_q > 1
    # leading dimensions: the mask may vary over a prefix of them and be shared by the rest
    varying = [i for i, d in enumerate(lead) if d > 1 and m.shape[i] == d]
    shared = [i for i, d in enumerate(lead) if d > 1 and m.shape[i] == 1]
    prefix_ok = not varying or not shared or max(varying) < min(shared)
    if m.shape[-1] != seq_k or not prefix_ok:
        m = m.expand(full).contiguous()
        return m, _ptr(m), 1, seq_q * seq_k, seq_k
    div = 1
    for i in shared:
        div *= lead[i]
    m = m.contiguous()
    row_stride = 0 if rows_shared else seq_k
    per_item = seq_k if rows_shared else m.shape[-2] * seq_k
    batch_stride = per_item if varying else 0
    return m, _ptr(m), div, batch_stride, row_stride


def attention(lut, q, k, v, divisor, mask=None):
    """DotProductAttention.call on ``[..., seq, depth]`` operands with identical leading
    dimensions: returns (out, weights).  Both products go through the LUT; the division by
    ``divisor``, the mask term and the softmax are plain FP32."""
    q, k, v = _dev(q, "queries"), _dev(k, "keys"), _dev(v, "values")
    lut = _lut(lut)
    if q.dim() < 2 or q.dim() != k.dim() or q.dim() != v.dim() or q.shape[:-2] != k.shape[:-2] or q.shape[:-2] != v.shape[:-2]:
        raise ValueError("queries, keys and values need identical leading dimensions")
    lead = tuple(q.shape[:-2])
    sq, dk = q.shape[-2:]
    sk, dk2 = k.shape[-2:]
    sk2, dv = v.shape[-2:]
    if dk != dk2 or sk != sk2:
        raise ValueError("keys must match the queries' depth and the values' length")
    batch = 1
    for d in lead:
        batch *= d
    keep, mptr, mdiv, mbs, mrs = _mask_layout(mask, lead, sq, sk, q.device)
    weights = torch.empty(lead + (sq, sk), dtype=torch.float32, device=q.device)
    out = torch.empty(lead + (sq, dv), dtype=torch.float32, device=q.device)
    lib = load_library()
    nbytes = lib.amsim_attention_workspace_bytes_for(lut.handle, batch, sq, sk, dk, dv)
    ws, wsp = _workspace(nbytes, q.device)
    check(lib.amsim_attention_f32(lut.handle, _ptr(q), _ptr(k), _ptr(v), mptr, mdiv, mbs, mrs, batch, sq, sk, dk, dv,
                                  float(divisor), _ptr(weights), _ptr(out), wsp, nbytes, _stream()))
    return out, weights


def attention_grad(lut, q, k, v, weights, grad_out, divisor):
    """Gradients of ``attention`` with respect to queries, keys and values."""
    q, k, v = _dev(q, "queries"), _dev(k, "keys"), _dev(v, "values")
    weights, grad_out = _dev(weights, "weights"), _dev(grad_out, "grad_out")
    lut = _lut(lut)
    lead = tuple(q.shape[:-2])
    sq, dk = q.shape[-2:]
    sk, dv = v.shape[-2:]
    batch = 1
    for d in lead:
        batch *= d
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    lib = load_library()
    nbytes = lib.amsim_attention_grad_workspace_bytes_for(lut.handle, batch, sq, sk, dk, dv)
    ws, wsp = _workspace(nbytes, q.device)
    check(lib.amsim_attention_grad_f32(lut.handle, _ptr(q), _ptr(k), _ptr(v), _ptr(weights), _ptr(grad_out), batch,
                                       sq, sk, dk, dv, float(divisor), _ptr(gq), _ptr(gk), _ptr(gv), wsp, nbytes,
                                       _stream()))
    return gq, gk, gv
