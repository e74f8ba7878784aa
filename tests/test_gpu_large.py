"""Operands beyond 2^31 elements (8 GiB of FP32) and tensors just below the
convolution entry points' 2^31-element limit: offsets must be formed in 64
bits on every path (dense staging along rows, dense staging along the
reduction, patch gathering, output stores).  The whole result cannot be
recomputed on the CPU in seconds, so slices whose addresses lie past the 2^31-
element and 2^32-byte marks are checked against the oracle, bit for bit."""
import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, host, lut32
from tests.util import lut_path

pytestmark = pytest.mark.gpu


def _needs_memory(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory")


def _bits_equal(got, want):
    return np.array_equal(np.ascontiguousarray(got).view(np.uint32), np.ascontiguousarray(want).view(np.uint32))


@pytest.fixture
def unsplit():
    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(0)
    yield
    lib.amsim_set_split_k(1)


def test_gemm_lane_operand_beyond_2_31_elements(unsplit):
    """A[M, K] with M*K > 2^31: rows near the end start past element 2^31."""
    from approxtrain_amd import ApproxMulLut, functors
    _needs_memory(12)
    M, K, N = (1 << 22) + 37, 520, 24
    assert M * K > (1 << 31)
    g = torch.Generator(device="cuda").manual_seed(41)
    A = torch.randn(M, K, device="cuda", generator=g)
    B = torch.randn(K, N, device="cuda", generator=g)
    out = functors.gemm(ApproxMulLut.cached(lut_path("MBM", 7)), A, B)
    torch.cuda.synchronize()
    assert out.shape == (M, N)
    L, Bh = lut32("MBM", 7), host(B)
    first_past_2_31 = (1 << 31) // K
    first_past_4g_bytes = (1 << 30) // K
    for lo in (0, first_past_4g_bytes - 3, first_past_2_31 - 3, M - 70):
        rows = slice(lo, min(lo + 70, M))
        assert _bits_equal(host(out[rows]), cpu.gemm(L, 7, host(A[rows]), Bh)), f"rows from {lo}"
    del A, out
    torch.cuda.empty_cache()


def test_gemm_reduction_beyond_2_31_elements():
    """dB = A^T . dC with A[K, M], K*M > 2^31: the reduction index walks past element
    2^31 of the lane operand.  Only the last rows of A are non-zero, so the oracle on
    that slice gives the whole result (a zero term adds +0 to a partial sum)."""
    from approxtrain_amd import ApproxMulLut, functors
    _needs_memory(40)
    K, M, N = (1 << 25) + 64, 64, 16
    assert K * M > (1 << 31)
    tail = 777
    g = torch.Generator(device="cuda").manual_seed(42)
    A = torch.zeros(K, M, device="cuda")
    A[K - tail:] = torch.randn(tail, M, device="cuda", generator=g)
    dC = torch.randn(K, N, device="cuda", generator=g)
    out = functors.gemm(ApproxMulLut.cached(lut_path("MBM", 7)), A, dC, trans_a=True)
    torch.cuda.synchronize()
    L = lut32("MBM", 7)
    At, Ct = host(A[K - tail:]), host(dC[K - tail:])
    want = cpu.gemm(L, 7, At, Ct, transA=True)
    assert_close_sum_abs(host(out), want, cpu.gemm_abs(L, 7, At, Ct, transA=True))
    del A, dC, out
    torch.cuda.empty_cache()


def test_conv_input_just_below_the_element_limit(unsplit):
    """NHWC input of 2^31 - 2^24 elements: the last image's patches lie at the top of
    the 32-bit element range the patch loader addresses with."""
    from approxtrain_amd import ApproxMulLut, functors
    _needs_memory(12)
    n, h, w, c, oc = 127, 512, 512, 64, 8
    assert (1 << 31) - (1 << 25) <= n * h * w * c < (1 << 31)
    g = torch.Generator(device="cuda").manual_seed(43)
    x = torch.randn(n, h, w, c, device="cuda", generator=g)
    filt = torch.randn(3, 3, c, oc, device="cuda", generator=g) * 0.1
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    y = functors.convam(lut, x, filt, (1, 1), "SAME")
    torch.cuda.synchronize()
    assert y.shape == (n, h, w, oc)
    L, fh = lut32("MBM", 7), host(filt)
    for b in (0, n - 1):
        # the bottom rows of image b: row 0 of the slice sees zero padding in the
        # oracle and real data on the GPU, so compare from row 1 on
        xs = host(x[b:b + 1, h - 6:])
        want = cpu.conv2d_fwd(L, 7, xs, fh, (1, 1), "SAME", threads=cpu.max_threads())
        assert _bits_equal(host(y[b, h - 5:]), want[0, 1:]), f"image {b}"
    del x, y
    torch.cuda.empty_cache()


def test_conv_gradients_just_below_the_element_limit():
    """Same tensor sizes through the two gradient passes.  Grad-filter reduces over every
    image: only the last one is non-zero, so the oracle on that image gives the whole sum.
    Grad-input stores 8 GiB of output: the bottom rows of the last image are checked."""
    from approxtrain_amd import ApproxMulLut, functors
    _needs_memory(40)
    n, h, w, c, oc = 127, 512, 512, 64, 8
    g = torch.Generator(device="cuda").manual_seed(44)
    x = torch.zeros(n, h, w, c, device="cuda")
    x[n - 1] = torch.randn(h, w, c, device="cuda", generator=g)
    dy = torch.randn(n, h, w, oc, device="cuda", generator=g)
    filt = torch.randn(3, 3, c, oc, device="cuda", generator=g) * 0.1
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    threads = cpu.max_threads()

    dw = functors.convam_filter_grad(lut, x, (3, 3, c, oc), dy, (1, 1), "SAME")
    torch.cuda.synchronize()
    xl, dyl = host(x[n - 1:]), host(dy[n - 1:])
    want = cpu.conv2d_grad_filter(L, 7, xl, (3, 3, c, oc), dyl, (1, 1), "SAME", threads=threads)
    sum_abs = cpu.conv2d_grad_filter(L, 7, np.abs(xl), (3, 3, c, oc), np.abs(dyl), (1, 1), "SAME", threads=threads)
    assert_close_sum_abs(host(dw), want, sum_abs)
    del x

    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(0)
    try:
        dx = functors.convam_input_grad(lut, (n, h, w, c), filt, dy, (1, 1), "SAME")
        torch.cuda.synchronize()
    finally:
        lib.amsim_set_split_k(1)
    assert dx.shape == (n, h, w, c)
    fh = host(filt)
    for b in (0, n - 1):
        dys = host(dy[b:b + 1, h - 6:])
        want = cpu.conv2d_grad_input(L, 7, (1, 6, w, c), fh, dys, (1, 1), "SAME", threads=threads)
        assert _bits_equal(host(dx[b, h - 5:]), want[0, 1:]), f"image {b}"
    del dx, dy
    torch.cuda.empty_cache()


def test_conv_rejects_inputs_of_2_31_elements():
    """At 2^31 elements the entry point refuses (status, no launch) instead of wrapping offsets."""
    import ctypes as C
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    n, h, w, c, oc = 128, 512, 512, 64, 8
    assert n * h * w * c == 1 << 31
    fake = C.c_void_p(256)  # never dereferenced: the size check comes first
    ws = lib.amsim_convam_workspace_bytes(n, h, w, oc, 3, 3, c)
    rc = lib.amsim_convam_f32(lut.handle, fake, fake, n, h, w, oc, 1, 1, 1, 1, 3, 3, c, w, h, fake, fake,
                              C.c_size_t(ws), None)
    assert rc != 0 and b"2^31" in lib.amsim_last_error()
