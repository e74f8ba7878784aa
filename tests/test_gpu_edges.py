"""Edge cases of the C-ABI entry points on the GPU: empty and ragged
extents, unaligned operands (scalar staging fallback), workspace errors,
large strides, reductions that are not multiples of the staging depth."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import dev, host, lut32
from tests.util import lut_path

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("amsim_engine")]


@pytest.fixture(autouse=True)
def _unsplit():
    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(0)
    yield
    lib.amsim_set_split_k(1)


def test_empty_extents_return_empty_outputs():
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    z = lambda *s: torch.zeros(*s, device="cuda")
    assert functors.gemm(lut, z(0, 5), z(5, 3)).shape == (0, 3)
    assert functors.gemm(lut, z(4, 5), z(5, 0)).shape == (4, 0)
    out = functors.gemm(lut, z(4, 0), z(0, 3))
    assert out.shape == (4, 3) and float(out.abs().sum()) == 0.0
    assert functors.convam(lut, z(0, 8, 8, 4), z(3, 3, 4, 5), (1, 1), "SAME").shape == (0, 8, 8, 5)
    assert functors.convam(lut, z(2, 2, 2, 4), z(3, 3, 4, 5), (1, 1), "VALID").shape == (2, 0, 0, 5)  # filter larger than input
    assert functors.convam_input_grad(lut, (0, 8, 8, 4), z(3, 3, 4, 5), z(0, 8, 8, 5), (1, 1), "SAME").shape == (0, 8, 8, 4)
    dw = functors.convam_filter_grad(lut, z(0, 8, 8, 4), (3, 3, 4, 5), z(0, 8, 8, 5), (1, 1), "SAME")
    assert dw.shape == (3, 3, 4, 5) and float(dw.abs().sum()) == 0.0  # empty reduction -> zeros
    assert functors.denseam(lut, z(0, 7), z(7, 3)).shape == (0, 3)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (63, 15, 31), (65, 17, 33), (64, 16, 32), (129, 1, 95), (2, 300, 3)])
def test_ragged_extents(M, N, K):
    from approxtrain_amd import ApproxMulLut, functors
    rng = np.random.default_rng(M + N + K)
    A, B = rng.standard_normal((M, K)).astype(np.float32), rng.standard_normal((K, N)).astype(np.float32)
    got = host(functors.gemm(ApproxMulLut.cached(lut_path("MBM", 7)), dev(A), dev(B)))
    assert np.array_equal(got.view(np.uint32), cpu.gemm(lut32("MBM", 7), 7, A, B).view(np.uint32))


def test_unaligned_operands_use_scalar_staging():
    """Operands that start 4 bytes into an allocation are not 16-byte aligned:
    the float4 staging path must not be taken (and results stay bit-equal)."""
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    rng = np.random.default_rng(5)
    M, N, K = 96, 48, 64
    A, B = rng.standard_normal((M, K)).astype(np.float32), rng.standard_normal((K, N)).astype(np.float32)
    buf = torch.zeros(M * K + 1, device="cuda")
    buf[1:] = dev(A).flatten()
    Au = buf[1:].view(M, K)
    assert Au.data_ptr() % 16 != 0 and Au.is_contiguous()
    got = host(functors.gemm(lut, Au, dev(B)))
    assert np.array_equal(got.view(np.uint32), cpu.gemm(L, 7, A, B).view(np.uint32))
    xs, ws = (2, 6, 6, 8), (3, 3, 8, 12)
    x, w = rng.standard_normal(xs).astype(np.float32), rng.standard_normal(ws).astype(np.float32)
    xb = torch.zeros(int(np.prod(xs)) + 1, device="cuda")
    xb[1:] = dev(x).flatten()
    xu = xb[1:].view(*xs)
    got = host(functors.convam(lut, xu, dev(w), (1, 1), "SAME"))
    assert np.array_equal(got.view(np.uint32), cpu.conv2d_fwd(L, 7, x, w, (1, 1), "SAME").view(np.uint32))


def test_leading_dimension_larger_than_row_and_workspace_errors():
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    rng = np.random.default_rng(6)
    M, N, K, lda, ldb, ldc = 70, 20, 40, 48, 28, 24
    A = rng.standard_normal((M, lda)).astype(np.float32)
    B = rng.standard_normal((K, ldb)).astype(np.float32)
    Ad, Bd = dev(A), dev(B)
    Cd = torch.full((M, ldc), 7.0, device="cuda")
    nbytes = lib.amsim_gemm_workspace_bytes(0, 0, M, N, K, 1)
    ws = torch.empty(nbytes + 512, dtype=torch.uint8, device="cuda")
    base = ws.data_ptr() + (-ws.data_ptr()) % 256
    args = lambda wsp, wsb: (lut.handle, 0, 0, 0, M, N, K, C.c_void_p(Ad.data_ptr()), lda, C.c_void_p(Bd.data_ptr()),
                             ldb, C.c_void_p(Cd.data_ptr()), ldc, 1, 0, 0, 0, C.c_void_p(wsp), wsb, None)
    assert lib.amsim_gemm_f32(*args(base, nbytes)) == 0
    got = host(Cd)
    want = cpu.gemm(lut32("MBM", 7), 7, A[:, :K].copy(), B[:, :N].copy())
    assert np.array_equal(got[:, :N].view(np.uint32), want.view(np.uint32))
    assert (got[:, N:] == 7.0).all()  # padding columns of C untouched
    assert lib.amsim_gemm_f32(*args(base, nbytes - 1)) == 5        # too small
    assert lib.amsim_gemm_f32(*args(base + 4, nbytes)) == 5        # misaligned
    assert lib.amsim_gemm_f32(*args(0, 0)) == 5                    # missing
    assert b"workspace" in lib.amsim_last_error()
    bad = list(args(base, nbytes)); bad[8] = K - 1                 # lda < K
    assert lib.amsim_gemm_f32(*bad) == 1


@pytest.mark.parametrize("stride", [3, 4])
def test_conv_large_strides_and_asymmetric_shapes(stride):
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(lut_path("MIT", 7))
    L = lut32("MIT", 7)
    rng = np.random.default_rng(stride)
    xs, ws = (2, 17, 13, 4), (5, 2, 4, 9)
    x, w = rng.standard_normal(xs).astype(np.float32), rng.standard_normal(ws).astype(np.float32)
    for padding in ("SAME", "VALID"):
        st = (stride, stride)
        want = cpu.conv2d_fwd(L, 7, x, w, st, padding)
        dy = rng.standard_normal(want.shape).astype(np.float32)
        assert np.array_equal(host(functors.convam(lut, dev(x), dev(w), st, padding)).view(np.uint32), want.view(np.uint32))
        assert np.array_equal(host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding)).view(np.uint32),
                              cpu.conv2d_grad_input(L, 7, xs, w, dy, st, padding).view(np.uint32))
        assert np.array_equal(host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding)).view(np.uint32),
                              cpu.conv2d_grad_filter(L, 7, x, ws, dy, st, padding).view(np.uint32))


def test_runs_on_a_non_default_stream():
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    rng = np.random.default_rng(9)
    A, B = rng.standard_normal((200, 96)).astype(np.float32), rng.standard_normal((96, 80)).astype(np.float32)
    s = torch.cuda.Stream()
    Ad, Bd = dev(A), dev(B)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        out = functors.gemm(lut, Ad, Bd)
    s.synchronize()
    assert np.array_equal(host(out).view(np.uint32), cpu.gemm(lut32("MBM", 7), 7, A, B).view(np.uint32))


def test_two_host_threads_on_two_streams_with_their_own_handles():
    """Calls are re-entrant: two host threads, each with its own stream, LUT handle (one keeps
    reductions whole, the other lets them be split) and workspaces, interleave convolution and GEMM
    calls; every result equals the one the same call gives alone."""
    from concurrent.futures import ThreadPoolExecutor
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    rng = np.random.default_rng(21)
    xs, ws = (4, 20, 20, 16), (3, 3, 16, 24)
    x, w = dev(rng.standard_normal(xs).astype(np.float32)), dev(rng.standard_normal(ws).astype(np.float32))
    dy = dev(rng.standard_normal((4, 20, 20, 24)).astype(np.float32))
    A, B = dev(rng.standard_normal((300, 700)).astype(np.float32)), dev(rng.standard_normal((700, 90)).astype(np.float32))
    luts = [ApproxMulLut(lut_path("MBM", 7)), ApproxMulLut(lut_path("MIT", 7))]
    assert lib.amsim_lut_set_split_k(luts[0].handle, 0) == 0 and lib.amsim_lut_set_split_k(luts[1].handle, 1) == 0

    def calls(lut):
        return [functors.convam(lut, x, w, (1, 1), "SAME"), functors.convam_input_grad(lut, xs, w, dy, (1, 1), "SAME"),
                functors.convam_filter_grad(lut, x, ws, dy, (1, 1), "SAME"), functors.gemm(lut, A, B),
                functors.gemm(lut, A, A, trans_b=True)]

    alone = [[host(t) for t in calls(lut)] for lut in luts]
    torch.cuda.synchronize()

    def worker(i):
        s = torch.cuda.Stream()
        outs = []
        with torch.cuda.stream(s):
            for _ in range(8):
                outs = calls(luts[i])
        s.synchronize()
        return [host(t) for t in outs]

    with ThreadPoolExecutor(max_workers=2) as pool:
        together = list(pool.map(worker, (0, 1)))
    for i in range(2):
        for got, want in zip(together[i], alone[i]):
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("xs,ws,stride,padding", [((2, 9, 8, 16), (1, 1, 16, 24), 2, "SAME"),     # taps reach 1 pixel in 4
                                                   ((2, 11, 7, 4), (2, 2, 4, 6), 3, "VALID"),      # filter smaller than stride
                                                   ((1, 12, 12, 32), (3, 3, 32, 32), 2, "SAME"),
                                                   ((3, 10, 13, 8), (5, 3, 8, 12), (2, 3), "SAME")])
def test_strided_grad_input_residue_classes(xs, ws, stride, padding):
    """Grad-input with strides above 1 runs one sub-problem per residue class of the input pixels:
    same bits as the oracle's dilated-gradient loop nest, zeros where no tap reaches."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    approxtrain_amd.load_library().amsim_set_split_k(0)
    try:
        lut = ApproxMulLut.cached(lut_path("MBM", 7))
        L = lut32("MBM", 7)
        st = (stride, stride) if isinstance(stride, int) else stride
        rng = np.random.default_rng(sum(xs))
        w = rng.standard_normal(ws).astype(np.float32)
        oh, _ = cpu.conv_geometry(xs[1], ws[0], st[0], padding)
        ow, _ = cpu.conv_geometry(xs[2], ws[1], st[1], padding)
        dy = rng.standard_normal((xs[0], oh, ow, ws[3])).astype(np.float32)
        got = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding))
        want = cpu.conv2d_grad_input(L, 7, xs, w, dy, st, padding)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        approxtrain_amd.load_library().amsim_set_split_k(1)


def test_strided_grad_input_with_the_stride_agnostic_workspace():
    """A caller that sizes the workspace with the reference-shaped query (no strides) still gets the
    right answer: sub-problems that would want more room run with their reductions whole."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lib.amsim_set_split_k(1)  # splitting allowed: the two workspace sizes then lead to different plans
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    n, h, w_, c, kh, kw, oc, s = 4, 28, 28, 64, 3, 3, 64, 2
    oh = ow = 14
    rng = np.random.default_rng(12)
    filt = rng.standard_normal((kh, kw, c, oc)).astype(np.float32)
    dy = rng.standard_normal((n, oh, ow, oc)).astype(np.float32)
    small = lib.amsim_convam_input_grad_workspace_bytes(n, h, w_, c, kh, kw, oc)
    big = lib.amsim_convam_input_grad_strided_workspace_bytes(n, h, w_, c, kh, kw, oc, s, s, kh - 1 - 0, kw - 1 - 0)
    assert big >= small
    outs = []
    for nbytes in (small, big):
        ws = torch.empty(nbytes + 512, dtype=torch.uint8, device="cuda")
        base = ws.data_ptr() + (-ws.data_ptr()) % 256
        out = torch.full((n, h, w_, c), 7.0, device="cuda")
        fd, gd = dev(filt), dev(dy)
        # SAME, stride 2, 28 -> 14: total padding 1, forward pad_top = 0 -> back pad = kh - 1
        rc = lib.amsim_convam_input_grad_f32(lut.handle, C.c_void_p(gd.data_ptr()), (ow - 1) * s + 1, (oh - 1) * s + 1,
                                             kh - 1, kw - 1, C.c_void_p(fd.data_ptr()), kh, kw, oc, s, s, n, h, w_, c,
                                             C.c_void_p(out.data_ptr()), oh, ow, C.c_void_p(base), nbytes, None)
        assert rc == 0, lib.amsim_last_error()
        outs.append(host(out))
    want = cpu.conv2d_grad_input(lut32("MBM", 7), 7, (n, h, w_, c), filt, dy, (s, s), "SAME")
    sum_abs = np.abs(want).max() * 50 + 1.0
    for got in outs:
        assert np.all(np.abs(got - want) <= 1e-5 * sum_abs)


@pytest.mark.parametrize("xs,ws,stride,padding,bad", [
    ((2, 9, 8, 5), (3, 3, 5, 4), (2, 2), "SAME", np.inf),
    ((1, 12, 7, 3), (3, 5, 3, 6), (3, 2), "VALID", np.nan),
    ((2, 10, 10, 16), (1, 1, 16, 8), (2, 2), "VALID", -np.inf),   # 1x1: three of four classes skip the only tap
    ((1, 7, 9, 4), (2, 2, 4, 3), (1, 3), "SAME", np.nan),
])
def test_strided_grad_input_with_non_finite_filter_weights(xs, ws, stride, padding, bad):
    """The reference multiplies every tap with the dilated gradient, inserted zeros included
    (cuda_kernel.cu:463-502): a weight that is inf or NaN turns 0 x w into NaN for every input
    pixel, not only for the pixels whose residue class meets that tap.  The residue-class
    sub-problems must reproduce that (NaNs compared as a class)."""
    from approxtrain_amd import ApproxMulLut, functors
    from tests.util import same_bits_or_both_nan
    lut, L = ApproxMulLut.cached(lut_path("MBM", 7)), lut32("MBM", 7)
    rng = np.random.default_rng(31)
    w = rng.standard_normal(ws).astype(np.float32)
    w[ws[0] - 1, 0, 1, 0] = bad          # one tap, one input channel
    oh, _ = cpu.conv_geometry(xs[1], ws[0], stride[0], padding)
    ow, _ = cpu.conv_geometry(xs[2], ws[1], stride[1], padding)
    dy = rng.standard_normal((xs[0], oh, ow, ws[3])).astype(np.float32)
    got = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), stride, padding))
    want = cpu.conv2d_grad_input(L, 7, xs, w, dy, stride, padding)
    assert np.all(same_bits_or_both_nan(got, want))
    assert np.isnan(want[..., 1]).any() and np.isfinite(want[..., 0]).all()   # only that channel is hit


def test_library_loaded_before_torch_still_shares_its_runtime():
    """A process that loads libamsim.so before it imports torch must not end up with two HIP
    runtimes (torch bundles its own copy; the second one to start finds no device)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import approxtrain_amd\n"
        "lib = approxtrain_amd.load_library()\n"            # before anything imports torch explicitly
        "import torch\n"
        "from approxtrain_amd import functors\n"
        "a = torch.ones(8, 16, device='cuda'); b = torch.ones(16, 4, device='cuda')\n"
        "out = functors.gemm('tests/golden/lut/ACC_7.bin', a, b)\n"
        "print('sum', float(out.sum()))\n")
    run = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "sum 512.0" in run.stdout


def test_per_handle_engine_and_reduction_settings_override_the_process_defaults():
    """Two handles of one table with different settings in one process: each call follows its own
    handle (amsim_lut_set_engine / amsim_lut_set_split_k), whatever the process-wide defaults say."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    a, b = ApproxMulLut(lut_path("MBM", 7)), ApproxMulLut(lut_path("MBM", 7))
    assert lib.amsim_lut_set_engine(a.handle, 1) == 0 and lib.amsim_lut_set_split_k(a.handle, 0) == 0   # LDS-table engine, whole reductions
    assert lib.amsim_lut_set_engine(b.handle, 2) == 0 and lib.amsim_lut_set_split_k(b.handle, 0) == 0   # direct engine, whole reductions
    assert lib.amsim_lut_set_engine(a.handle, 3) == 1 and lib.amsim_lut_set_split_k(a.handle, 2) == 1   # refused values
    rng = np.random.default_rng(21)
    A = rng.standard_normal((70, 4000)).astype(np.float32)
    B = rng.standard_normal((4000, 20)).astype(np.float32)
    want = cpu.gemm(lut32("MBM", 7), 7, A, B)
    lib.amsim_set_split_k(1)  # the default would split this long reduction over workgroups
    for lut in (a, b):
        got = host(functors.gemm(lut, dev(A), dev(B)))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
