"""ctypes bindings of oracle/liboracle.so (built by oracle/Makefile) and, when
it was built in the container that holds the reference tree, of
oracle/_ref/libref_models.so (the reference's own C functional models).

TEST INFRASTRUCTURE: the checker, never the thing measured or shipped.
"""
import ctypes as C
import os
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_F = C.POINTER(C.c_float)
_U32 = C.POINTER(C.c_uint32)
_U8 = C.POINTER(C.c_uint8)

KIND = {"MBM": 0, "MIT": 1, "ACC": 2}


def _load(path):
    if not os.path.exists(path):
        raise FileNotFoundError(f"{path} missing: run `make -C oracle`")
    return C.CDLL(path)


_lib = _load(os.path.join(_HERE, "liboracle.so"))
_lib.amo_model.restype = C.c_float
_lib.amo_model.argtypes = [C.c_int, C.c_int, C.c_float, C.c_float]
_lib.amo_lut_mul.restype = C.c_float
_lib.amo_max_threads.restype = C.c_int


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_F)


def _lut(lut32):
    assert lut32.dtype == np.uint32 and lut32.flags.c_contiguous
    return lut32.ctypes.data_as(_U32)


def max_threads():
    return int(_lib.amo_max_threads())


def model_array(kind, m, a, b):
    """Functional model `kind` ('MBM' | 'MIT' | 'ACC') at mantissa width m."""
    a, pa = _f(a)
    b, pb = _f(b)
    out = np.empty_like(a)
    _lib.amo_model_array(C.c_int(KIND[kind]), C.c_int(m), pa, pb, out.ctypes.data_as(_F), C.c_long(a.size))
    return out


def lutgen(kind, m):
    out = np.zeros(1 << (2 * m), dtype=np.uint8)
    rc = _lib.amo_lutgen(C.c_int(KIND[kind]), C.c_int(m), out.ctypes.data_as(_U8))
    if rc != 0:
        raise ValueError("amo_lutgen: m out of range")
    return out


def lutgen32(kind, m):
    out = np.zeros(1 << (2 * m), dtype=np.uint32)
    rc = _lib.amo_lutgen32(C.c_int(KIND[kind]), C.c_int(m), out.ctypes.data_as(_U32))
    if rc != 0:
        raise ValueError("amo_lutgen32: bad kind/m")
    return out


def expand_u8(lut8, m):
    lut8 = np.ascontiguousarray(lut8, dtype=np.uint8)
    assert lut8.size == 1 << (2 * m)
    out = np.zeros(lut8.size, dtype=np.uint32)
    _lib.amo_expand_u8(lut8.ctypes.data_as(_U8), C.c_int(m), out.ctypes.data_as(_U32))
    return out


def lut_mul_array(lut32, m, a, b):
    a, pa = _f(a)
    b, pb = _f(b)
    out = np.empty_like(a)
    _lib.amo_lut_mul_array(_lut(lut32), C.c_int(m), pa, pb, out.ctypes.data_as(_F), C.c_long(a.size))
    return out


def gemm(lut32, m, A, B, transA=False, transB=False, swap=False, threads=1):
    """C = op(A) . op(B) with the LUT product, FP32 ascending-k accumulation."""
    A, pa = _f(A)
    B, pb = _f(B)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    K2, N = (B.shape[1], B.shape[0]) if transB else B.shape
    assert K == K2
    out = np.zeros((M, N), dtype=np.float32)
    _lib.amo_gemm(_lut(lut32), C.c_int(m), C.c_int(transA), C.c_int(transB), C.c_int(swap),
                  C.c_long(M), C.c_long(N), C.c_long(K), pa, C.c_long(A.shape[1]), pb,
                  C.c_long(B.shape[1]), out.ctypes.data_as(_F), C.c_long(N), C.c_int(threads))
    return out


def gemm_abs(lut32, m, A, B, transA=False, transB=False, swap=False, threads=1):
    """sum_k |P(a,b)| per output, in float64: the tolerance normaliser."""
    A, pa = _f(A)
    B, pb = _f(B)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    K2, N = (B.shape[1], B.shape[0]) if transB else B.shape
    assert K == K2
    out = np.zeros((M, N), dtype=np.float64)
    _lib.amo_gemm_abs(_lut(lut32), C.c_int(m), C.c_int(transA), C.c_int(transB), C.c_int(swap),
                      C.c_long(M), C.c_long(N), C.c_long(K), pa, C.c_long(A.shape[1]), pb,
                      C.c_long(B.shape[1]), out.ctypes.data_as(C.POINTER(C.c_double)), C.c_long(N), C.c_int(threads))
    return out


def dense_fwd(lut32, m, x, w):
    x, px = _f(x)
    w, pw = _f(w)
    batch, iw = x.shape
    units = w.shape[1]
    y = np.zeros((batch, units), dtype=np.float32)
    _lib.amo_dense_fwd(_lut(lut32), C.c_int(m), px, pw, y.ctypes.data_as(_F), C.c_int(batch), C.c_int(units), C.c_int(iw))
    return y


def dense_grad(lut32, m, dy, x, w):
    """Returns (grad_input, grad_weights) like the DenseamGrad op."""
    x, px = _f(x)
    w, pw = _f(w)
    dy, pdy = _f(dy)
    batch, iw = x.shape
    units = w.shape[1]
    dw = np.zeros_like(w)
    dx = np.zeros_like(x)
    _lib.amo_dense_grad_w(_lut(lut32), C.c_int(m), px, pdy, dw.ctypes.data_as(_F), C.c_int(batch), C.c_int(units), C.c_int(iw))
    _lib.amo_dense_grad_x(_lut(lut32), C.c_int(m), pw, pdy, dx.ctypes.data_as(_F), C.c_int(batch), C.c_int(units), C.c_int(iw))
    return dx, dw


def conv_geometry(in_size, k, stride, padding):
    """TensorFlow 2.3 GetWindowedOutputSizeVerbose, closed form (dilation 1):
    VALID o = ceil((i-k+1)/s), pad 0; SAME o = ceil(i/s),
    pad_before = max((o-1)s + k - i, 0) // 2."""
    if padding == "VALID":
        return (in_size - k + stride) // stride, 0
    o = (in_size + stride - 1) // stride
    return o, max((o - 1) * stride + k - in_size, 0) // 2


def _conv_args(x_shape, w_shape, strides, padding):
    n, h, w_, c = x_shape
    kh, kw, c2, oc = w_shape
    assert c == c2
    oh, pt = conv_geometry(h, kh, strides[0], padding)
    ow, pl = conv_geometry(w_, kw, strides[1], padding)
    ints = [n, h, w_, c, kh, kw, oc, strides[0], strides[1], pt, pl, oh, ow]
    return [C.c_int(v) for v in ints], (n, oh, ow, oc)


def conv2d_fwd(lut32, m, x, w, strides=(1, 1), padding="SAME", threads=1):
    x, px = _f(x)
    w, pw = _f(w)
    args, oshape = _conv_args(x.shape, w.shape, strides, padding)
    y = np.zeros(oshape, dtype=np.float32)
    _lib.amo_conv2d_fwd(_lut(lut32), C.c_int(m), px, pw, y.ctypes.data_as(_F), *args, C.c_int(threads))
    return y


def conv2d_grad_filter(lut32, m, x, w_shape, dy, strides=(1, 1), padding="SAME", threads=1):
    x, px = _f(x)
    dy, pdy = _f(dy)
    args, oshape = _conv_args(x.shape, w_shape, strides, padding)
    assert tuple(dy.shape) == oshape
    dw = np.zeros(w_shape, dtype=np.float32)
    _lib.amo_conv2d_grad_filter(_lut(lut32), C.c_int(m), px, pdy, dw.ctypes.data_as(_F), *args, C.c_int(threads))
    return dw


def conv2d_grad_input(lut32, m, x_shape, w, dy, strides=(1, 1), padding="SAME", threads=1):
    w, pw = _f(w)
    dy, pdy = _f(dy)
    args, oshape = _conv_args(x_shape, w.shape, strides, padding)
    assert tuple(dy.shape) == oshape
    dx = np.zeros(x_shape, dtype=np.float32)
    _lib.amo_conv2d_grad_input(_lut(lut32), C.c_int(m), pdy, pw, dx.ctypes.data_as(_F), *args, C.c_int(threads))
    return dx


def matmul(lut32, m, a, b):
    """MatMulAM shape cases: rank 2/3 operands, batch broadcast of size 1."""
    a, pa = _f(a)
    b, pb = _f(b)
    ba = a.shape[0] if a.ndim == 3 else 0
    bb = b.shape[0] if b.ndim == 3 else 0
    ra, ca = a.shape[-2:]
    rb, cb = b.shape[-2:]
    nb = max(ba, bb)
    out = np.zeros((nb, ra, cb) if nb else (ra, cb), dtype=np.float32)
    rc = _lib.amo_matmul(_lut(lut32), C.c_int(m), pa, pb, C.c_int(ba), C.c_int(bb), C.c_int(ra),
                         C.c_int(ca), C.c_int(rb), C.c_int(cb), out.ctypes.data_as(_F))
    if rc != 0:
        raise ValueError("matmul: incompatible shapes")
    return out


# --- the reference's own compiled functional models (oracle/_ref) -----------
_REF_FUNCS = {
    ("MBM", 7): "FPmultMBM_fast16", ("MBM", 5): "FPmultMBM_fast14",
    ("MBM", 3): "FPmultMBM_fast12", ("MBM", 1): "FPmultMBM_fast10",
    ("MIT", 7): "FPmultMitch_fast16", ("MIT", 5): "FPmultMitch_fast14",
    ("MIT", 3): "FPmultMitch_fast12", ("MIT", 1): "FPmultMitch_fast10",
    ("ACC", 7): "bfloat16mul",
}
_ref = None


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libref_models.so"))


def ref_model_array(kind, m, a, b):
    """The reference's compiled C model, swept over arrays by the shim's loop."""
    global _ref
    if _ref is None:
        _ref = _load(os.path.join(_HERE, "_ref", "libref_models.so"))
    fn = getattr(_ref, "ref_array_" + _REF_FUNCS[(kind, m)])
    a, pa = _f(a)
    b, pb = _f(b)
    out = np.empty_like(a)
    fn(pa, pb, out.ctypes.data_as(_F), C.c_long(a.size))
    return out
