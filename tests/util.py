"""Shared input generators for the parity tests."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LUT_FILES = [("MBM", 1), ("MBM", 3), ("MBM", 5), ("MBM", 7),
             ("MIT", 1), ("MIT", 3), ("MIT", 5), ("MIT", 7), ("ACC", 7)]


def lut_path(kind, m):
    return os.path.join(GOLDEN, "lut", f"{kind}_{m}.bin")


def lut_bytes(kind, m):
    return np.fromfile(lut_path(kind, m), dtype=np.uint8)


def bits(sign, exp, frac):
    return ((np.asarray(sign, np.uint32) << 31) | (np.asarray(exp, np.uint32) << 23)
            | np.asarray(frac, np.uint32)).astype(np.uint32)


def _low_bits(rng, n, m):
    """Fraction bits below the m kept ones: all-zero, all-one or random."""
    lowmask = (1 << (23 - m)) - 1
    mode = rng.integers(0, 3, n)
    low = rng.integers(0, lowmask + 1, n, dtype=np.uint32)
    low = np.where(mode == 0, 0, np.where(mode == 1, lowmask, low)).astype(np.uint32)
    return low


def product_domain(m, seed, reps=2):
    """Operand pairs (uint32 bit patterns) covering: every mantissa pair at
    random normal exponents and signs; every exponent pair (0..255)^2 with
    random mantissas; exponent sums around both range boundaries with every
    mantissa pair (sampled for m = 7); zeros, subnormals, infinities, NaNs
    against everything."""
    rng = np.random.default_rng(seed)
    A, B = [], []
    n = 1 << m

    def add(sa, ea, fa, sb, eb, fb):
        A.append(bits(sa, ea, fa))
        B.append(bits(sb, eb, fb))

    # 1. every mantissa pair, random exponents/signs/low bits
    ia, ib = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32), indexing="ij")
    ia, ib = ia.ravel(), ib.ravel()
    for _ in range(reps):
        k = ia.size
        add(rng.integers(0, 2, k), rng.integers(1, 255, k), (ia << (23 - m)) | _low_bits(rng, k, m),
            rng.integers(0, 2, k), rng.integers(1, 255, k), (ib << (23 - m)) | _low_bits(rng, k, m))
    # 2. every exponent pair, random mantissas
    ea, eb = np.meshgrid(np.arange(256, dtype=np.uint32), np.arange(256, dtype=np.uint32), indexing="ij")
    ea, eb = ea.ravel(), eb.ravel()
    for _ in range(4 * reps):
        k = ea.size
        add(rng.integers(0, 2, k), ea, rng.integers(0, 1 << 23, k, dtype=np.uint32),
            rng.integers(0, 2, k), eb, rng.integers(0, 1 << 23, k, dtype=np.uint32))
    # 3. exponent sums at the underflow / overflow boundaries x mantissa pairs
    if m == 7:
        sel = rng.choice(ia.size, 2048, replace=False)
        ja, jb = ia[sel], ib[sel]
    else:
        ja, jb = ia, ib
    for E in (125, 126, 127, 128, 129, 379, 380, 381, 382, 383):
        for e1 in (1, 60, 126, 127, 128, 200, 254):
            e2 = E - e1
            if not (1 <= e2 <= 254):
                continue
            k = ja.size
            add(rng.integers(0, 2, k), np.full(k, e1), (ja << (23 - m)) | _low_bits(rng, k, m),
                rng.integers(0, 2, k), np.full(k, e2), (jb << (23 - m)) | _low_bits(rng, k, m))
    # 4. specials against a spread of ordinary values and against each other
    spec = np.array([0x00000000, 0x80000000, 0x00000001, 0x807fffff, 0x00400000, 0x00012345,
                     0x7f800000, 0xff800000, 0x7fc00000, 0xffc00001, 0x7f800001,
                     0x00800000, 0x7f7fffff, 0x3f800000, 0xbf800000], dtype=np.uint32)
    k = 4096
    ordinary = bits(rng.integers(0, 2, k), rng.integers(0, 256, k), rng.integers(0, 1 << 23, k, dtype=np.uint32))
    for s in spec:
        A.append(np.full(k, s, np.uint32)); B.append(ordinary)
        A.append(ordinary); B.append(np.full(k, s, np.uint32))
    sa, sb = np.meshgrid(spec, spec, indexing="ij")
    A.append(sa.ravel()); B.append(sb.ravel())
    a = np.concatenate(A).astype(np.uint32)
    b = np.concatenate(B).astype(np.uint32)
    return a, b


def same_bits_or_both_nan(x, y):
    """Bit equality, except that any NaN matches any NaN (payload and quiet
    bit of a propagated NaN are implementation details of the multiplier)."""
    xb = np.asarray(x, np.float32).view(np.uint32)
    yb = np.asarray(y, np.float32).view(np.uint32)
    nan = np.isnan(np.asarray(x, np.float32)) & np.isnan(np.asarray(y, np.float32))
    return (xb == yb) | nan


# ---- shapes of the reference's own convolution test (test/convam_final_test.py:167-196)
# (N, H, W, C, KH, KW, C, OC); run there with strides 1 and 2, VALID and SAME.
REF_CONV_SHAPES = [
    (1, 4, 4, 1, 4, 4, 1, 1), (1, 4, 4, 1, 3, 3, 1, 1), (1, 4, 4, 1, 2, 2, 1, 1), (1, 4, 4, 1, 1, 1, 1, 1),
    (1, 4, 8, 1, 4, 4, 1, 1), (1, 4, 8, 1, 3, 3, 1, 1), (1, 4, 8, 1, 2, 2, 1, 1), (1, 4, 8, 1, 1, 1, 1, 1),
    (1, 4, 8, 1, 4, 5, 1, 1), (1, 4, 8, 1, 3, 4, 1, 1), (1, 4, 8, 1, 2, 1, 1, 1),
    (1, 4, 8, 2, 4, 5, 2, 3), (1, 4, 8, 2, 3, 4, 2, 3), (1, 4, 8, 2, 2, 1, 2, 3), (1, 4, 8, 2, 1, 1, 2, 3),
    (1, 8, 4, 3, 5, 4, 3, 4), (1, 8, 4, 3, 3, 4, 3, 4), (1, 8, 4, 3, 2, 1, 3, 4), (1, 8, 4, 3, 1, 1, 3, 4),
    (1, 20, 20, 3, 5, 5, 3, 4), (1, 20, 20, 3, 5, 4, 3, 4), (1, 20, 20, 3, 2, 1, 3, 4), (1, 20, 20, 3, 1, 1, 3, 4),
    (128, 32, 32, 1, 5, 5, 1, 6), (128, 14, 14, 6, 5, 5, 6, 16), (4, 4, 4, 1, 2, 2, 1, 2), (4, 14, 14, 1, 5, 5, 1, 16),
]


def tf_same_pads(in_size, k, stride):
    o = (in_size + stride - 1) // stride
    total = max((o - 1) * stride + k - in_size, 0)
    return o, total // 2, total - total // 2


def torch_conv_reference(x, w, dy, strides, padding):
    """Exact (float64) NHWC/HWIO convolution with TensorFlow's VALID/SAME
    geometry, and its autograd gradients for upstream gradient dy.
    Returns (y, dx, dw) as float64 numpy arrays. dy may be None."""
    import torch
    import torch.nn.functional as F
    xt = torch.tensor(np.asarray(x, np.float64)).permute(0, 3, 1, 2).contiguous().requires_grad_(True)
    wt = torch.tensor(np.asarray(w, np.float64)).permute(3, 2, 0, 1).contiguous().requires_grad_(True)
    if padding == "SAME":
        _, pt, pb = tf_same_pads(x.shape[1], w.shape[0], strides[0])
        _, pl, pr = tf_same_pads(x.shape[2], w.shape[1], strides[1])
        xp = F.pad(xt, (pl, pr, pt, pb))
    else:
        xp = xt
    y = F.conv2d(xp, wt, stride=tuple(strides))
    y_nhwc = y.permute(0, 2, 3, 1)
    if dy is None:
        return y_nhwc.detach().numpy(), None, None
    y_nhwc.backward(torch.tensor(np.asarray(dy, np.float64)))
    return (y_nhwc.detach().numpy(), xt.grad.permute(0, 2, 3, 1).numpy(),
            wt.grad.permute(2, 3, 1, 0).numpy())


def small_ints(rng, shape, lo=-8, hi=8):
    """Integer-valued float32 operands: with <= 3 fraction bits each, the
    truncated-exact (ACC_7) multiplier returns the exact product."""
    return rng.integers(lo, hi, size=shape).astype(np.float32)
