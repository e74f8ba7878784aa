"""Tables too wide for the LDS (mantissa widths 8..11) on the row-staged engine: problems with at
least 512 rows, through the C ABI, BIT-EQUAL to the CPU oracle where the reduction is kept whole (one
ascending-k FP32 chain per output), within 1e-5 * sum|products| where it may be sliced.

Parity note: no reference file or functional model exists above width 7.  The tables come from
the oracle's generator, i.e. from the closed-form rules that reproduce every reference file up to
width 7; beyond that rule the tables' parity is unpinned.  What these tests pin is that the GPU
multiplies and accumulates through whatever table it is given exactly like the oracle's loop nest
(cuda/gemm.cu:17-58 with the lookup of lut/AMsimulator.inl:18-23)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import dev, host
from tests.util import same_bits_or_both_nan

pytestmark = pytest.mark.gpu


def _legacy(img):
    return (((img >> 23) << 31) | (img & 0x7fffff)).astype(np.uint32)


@pytest.fixture(scope="module")
def luts():
    from approxtrain_amd import ApproxMulLut
    cache = {}

    def get(kind, m):
        if (kind, m) not in cache:
            import approxtrain_amd
            img = cpu.lutgen32(kind, m)
            lut = ApproxMulLut.from_entries(_legacy(img), m)
            # whole reductions for calls through these handles: every engine's result is then
            # bit-comparable with the oracle's
            assert approxtrain_amd.load_library().amsim_lut_set_split_k(lut.handle, 0) == 0
            cache[(kind, m)] = (lut, img)
        return cache[(kind, m)]
    return get


def _ops(rng, M, N, K, ta, tb):
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    A[rng.random(A.shape) < 0.1] = 0.0
    B[rng.random(B.shape) < 0.05] = 0.0
    return A, B


@pytest.mark.parametrize("kind,m", [("MBM", 11), ("MIT", 11), ("MBM", 10), ("MIT", 9), ("MBM", 8)])
@pytest.mark.parametrize("M,N,K,ta,tb", [(1100, 37, 70, 0, 0), (40, 2100, 64, 0, 0), (4200, 16, 33, 1, 0),
                                         (1030, 50, 96, 0, 1), (24, 1500, 40, 1, 1)])
def test_row_staged_gemm_bit_equal_to_oracle(luts, kind, m, M, N, K, ta, tb):
    from approxtrain_amd import functors
    lut, img = luts(kind, m)
    rng = np.random.default_rng(1000 * m + M + N + K + 2 * ta + tb)
    A, B = _ops(rng, M, N, K, ta, tb)
    got = host(functors.gemm(lut, dev(A), dev(B), trans_a=bool(ta), trans_b=bool(tb)))
    want = cpu.gemm(img, m, A, B, transA=ta, transB=tb)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("m", [11, 8])
def test_row_staged_gemm_full_domain_operands(luts, m):
    """Subnormals, infinities, NaN, huge and tiny magnitudes in either operand flag their
    32-deep chunk, which then takes the full-domain product; NaNs compare as a class."""
    from approxtrain_amd import functors
    lut, img = luts("MBM", m)
    rng = np.random.default_rng(5 + m)
    M, N, K = 1300, 40, 100
    A, B = _ops(rng, M, N, K, 0, 0)
    specials = np.array([1e-40, -1e-42, np.inf, -np.inf, np.nan, 3e38, -1e-38, 2.0 ** -70, 2.0 ** 70], np.float32)
    for s in specials:
        A[rng.integers(M), rng.integers(K)] = s
        B[rng.integers(K), rng.integers(N)] = s
    A[700, 40:72] = 2.0 ** 100   # a chunk flagged by the lane operand only
    B[64:96, 7] = 2.0 ** -100    # a chunk flagged by the uniform operand only
    got = host(functors.gemm(lut, dev(A), dev(B)))
    want = cpu.gemm(img, m, A, B)
    assert same_bits_or_both_nan(got, want).all()
    assert np.isnan(want).any() and np.isfinite(want).any()


def test_row_staged_gemm_operand_order_with_asymmetric_table(luts):
    """A table whose entry depends on which operand indexes its row: both LUT orientations
    (the two transposed device images) and the swap flag must agree with the oracle."""
    from approxtrain_amd import ApproxMulLut, functors
    m = 8
    n = 1 << m
    i, j = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32), indexing="ij")
    mant = (i * 3 + j * 5 + 1) % n
    img = (((i > j).astype(np.uint32) << 23) | (mant << (23 - m))).astype(np.uint32).ravel()
    lut = ApproxMulLut.from_entries(_legacy(img), m)
    rng = np.random.default_rng(8)
    A, B = _ops(rng, 1200, 30, 48, 0, 0)
    for swap in (False, True):
        got = host(functors.gemm(lut, dev(A), dev(B), swap_operands=swap))
        want = cpu.gemm(img, m, A, B, swap=swap)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # rows over N: the other device image serves the same product
    A2, B2 = _ops(rng, 20, 1400, 48, 0, 0)
    for swap in (False, True):
        got = host(functors.gemm(lut, dev(A2), dev(B2), swap_operands=swap))
        want = cpu.gemm(img, m, A2, B2, swap=swap)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dense_layer_with_fused_epilogue_on_row_staged_engine(luts):
    from approxtrain_amd import functors
    lut, img = luts("MIT", 11)
    rng = np.random.default_rng(12)
    x = rng.standard_normal((1500, 40)).astype(np.float32)
    w = rng.standard_normal((40, 24)).astype(np.float32)
    b = rng.standard_normal(24).astype(np.float32)
    got = host(functors.denseam(lut, dev(x), dev(w), bias=dev(b), activation="relu"))
    y = cpu.dense_fwd(img, 11, x, w) + b
    want = np.where(y < 0, np.float32(0), y).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_smaller_workspace_falls_back_to_global_gathers(luts):
    """The LUT-less workspace query covers the row-staged engine; a caller that brings only what
    the global-gather variant needs still gets the same bits."""
    import approxtrain_amd
    from approxtrain_amd._lib import check
    lib = approxtrain_amd.load_library()
    lut, img = luts("MBM", 11)
    rng = np.random.default_rng(13)
    M, N, K = 1100, 20, 64
    A, B = _ops(rng, M, N, K, 0, 0)
    Ad, Bd = dev(A), dev(B)
    full = lib.amsim_gemm_workspace_bytes(0, 0, M, N, K, 1)
    assert full > 4 * M * K   # holds the transposed lane operand
    small = 512 * 1024
    outs = []
    for nbytes in (full, small):
        ws = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda")
        wsp = C.c_void_p(ws.data_ptr() + (-ws.data_ptr()) % 256)
        out = torch.empty((M, N), device="cuda")
        check(lib.amsim_gemm_f32(lut.handle, 0, 0, 0, M, N, K, C.c_void_p(Ad.data_ptr()), K, C.c_void_p(Bd.data_ptr()), N,
                                 C.c_void_p(out.data_ptr()), N, 1, 0, 0, 0, wsp, nbytes, None))
        outs.append(host(out))
    want = cpu.gemm(img, 11, A, B)
    assert np.array_equal(outs[0].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(outs[1].view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("kind,m", [("MBM", 11), ("MIT", 9)])
@pytest.mark.parametrize("shape", [((2, 24, 26, 8), (3, 3, 8, 20), (1, 1), "SAME"),
                                   ((1, 40, 40, 3), (5, 4, 3, 7), (1, 1), "VALID"),
                                   ((3, 30, 30, 16), (3, 3, 16, 12), (2, 2), "SAME"),
                                   ((2, 33, 31, 4), (2, 3, 4, 9), (2, 1), "VALID")])
def test_convolution_forward_and_input_gradient_on_row_staged_engine(luts, kind, m, shape):
    """Wide tables through the convolution entry points: with the table-aware workspace query the
    forward pass and the input gradient (all its stride phases with 1024 or more pixels) gather from
    an im2col staged for the row-staged engine; bit-equal to the oracle's loop nests either way."""
    from approxtrain_amd import functors
    lut, img = luts(kind, m)
    xs, ws, st, padding = shape
    rng = np.random.default_rng(m * 100 + xs[1] + ws[0])
    x = rng.standard_normal(xs).astype(np.float32)
    x[rng.random(xs) < 0.3] = 0.0
    w = rng.standard_normal(ws).astype(np.float32)
    y = host(functors.convam(lut, dev(x), dev(w), st, padding))
    want = cpu.conv2d_fwd(img, m, x, w, st, padding)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    dy = rng.standard_normal(want.shape).astype(np.float32)
    dx = host(functors.convam_input_grad(lut, xs, dev(w), dev(dy), st, padding))
    want_dx = cpu.conv2d_grad_input(img, m, xs, w, dy, st, padding)
    assert np.array_equal(dx.view(np.uint32), want_dx.view(np.uint32))


@pytest.mark.parametrize("kind,m", [("MBM", 11), ("MIT", 8)])
@pytest.mark.parametrize("shape", [((2, 24, 26, 8), (3, 3, 8, 20), (1, 1), "SAME"),
                                   ((1, 40, 40, 3), (5, 4, 3, 7), (1, 1), "VALID"),
                                   ((3, 30, 30, 16), (3, 3, 16, 12), (2, 2), "SAME"),
                                   ((2, 33, 31, 40), (2, 3, 40, 9), (2, 1), "VALID"),
                                   ((9, 20, 20, 64), (3, 3, 64, 24), (1, 1), "SAME")])   # several row tiles, sliced reduction
def test_convolution_forward_from_the_channel_major_copy(luts, kind, m, shape):
    """The lean workspace tier: given the amount amsim_convam_lean_workspace_bytes_for returns --
    room for a zero-bordered channel-major copy of the input, not for an im2col -- the forward
    pass runs on the row-staged engine from that copy.  Bit-equal to the oracle with reductions
    kept whole, within 1e-5 * sum|products| with slices; a special value in the input takes the
    full-domain path of the tiles that can reach it."""
    import ctypes as C
    import torch
    import approxtrain_amd
    from approxtrain_amd._lib import check, conv_geometry
    from tests.gpu_util import assert_close_sum_abs
    from tests.util import torch_conv_reference
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    _, img = luts(kind, m)
    lut = ApproxMulLut.from_entries(_legacy(img), m)  # a handle of this test's own: it changes the split mode
    assert lib.amsim_lut_set_split_k(lut.handle, 1) == 0
    xs, ws, st, padding = shape
    rng = np.random.default_rng(m * 10 + xs[1] + ws[1])
    x = rng.standard_normal(xs).astype(np.float32)
    x[rng.random(xs) < 0.3] = 0.0
    w = rng.standard_normal(ws).astype(np.float32)
    n, h, wd, c = xs
    kh, kw, _, oc = ws
    oh, pt = conv_geometry(h, kh, st[0], padding)
    ow, pl = conv_geometry(wd, kw, st[1], padding)
    lean = lib.amsim_convam_lean_workspace_bytes_for(lut.handle, n, oh, ow, oc, kh, kw, c, st[0], st[1])
    full = lib.amsim_convam_workspace_bytes_for(lut.handle, n, oh, ow, oc, kh, kw, c)
    assert lib.amsim_convam_workspace_bytes(n, oh, ow, oc, kh, kw, c) <= lean
    if kh * kw >= 4:
        assert lean < full, "the copy must be smaller than the im2col"
    ws_t = torch.empty(lean + 256, dtype=torch.uint8, device="cuda")
    wsp = ws_t.data_ptr() + (-ws_t.data_ptr()) % 256
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(xa):
        xd, wdv = dev(xa), dev(w)
        out = torch.full((n, oh, ow, oc), float("nan"), dtype=torch.float32, device="cuda")
        check(lib.amsim_convam_f32(lut.handle, C.c_void_p(xd.data_ptr()), C.c_void_p(out.data_ptr()), n, oh, ow, oc, st[1], st[0],
                                   pl, pt, kh, kw, c, wd, h, C.c_void_p(wdv.data_ptr()), C.c_void_p(wsp), lean, stream))
        torch.cuda.synchronize()
        return host(out)

    want = cpu.conv2d_fwd(img, m, x, w, st, padding)
    s_y, _, _ = torch_conv_reference(np.abs(x), np.abs(w), None, st, padding)
    assert_close_sum_abs(run(x), want, s_y, 1e-5)
    assert lib.amsim_lut_set_split_k(lut.handle, 0) == 0
    assert np.array_equal(run(x).view(np.uint32), want.view(np.uint32))
    # special values: an infinity, a NaN, a subnormal and a huge value somewhere in the image
    xsp = x.copy()
    flat = xsp.reshape(-1)
    pos = rng.choice(flat.size, 4, replace=False)
    flat[pos] = np.array([np.inf, np.nan, 1e-41, 3e38], np.float32)
    want_sp = cpu.conv2d_fwd(img, m, xsp, w, st, padding)
    got_sp = run(xsp)
    from tests.util import same_bits_or_both_nan
    assert same_bits_or_both_nan(got_sp, want_sp).all()
    lut.close()


def test_table_aware_convolution_query_adds_the_staged_operand_only_for_wide_tables(luts):
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    from tests.util import lut_path
    lib = approxtrain_amd.load_library()
    wide, _ = luts("MBM", 11)
    narrow = ApproxMulLut(lut_path("MBM", 7))
    args = (4, 56, 56, 64, 3, 3, 64)
    base = lib.amsim_convam_workspace_bytes(*args)
    assert lib.amsim_convam_workspace_bytes_for(narrow.handle, *args) == base
    assert lib.amsim_convam_workspace_bytes_for(wide.handle, *args) >= (4 * 56 * 56) * 576 * 4   # rows x reduction x 4 bytes: the im2col
    assert lib.amsim_convam_workspace_bytes_for(None, *args) == base


def test_batched_products_on_row_staged_engine(luts):
    """Strided batches with 1024 or more rows per item, per-item and shared second operands."""
    from approxtrain_amd import functors
    lut, img = luts("MIT", 11)
    rng = np.random.default_rng(31)
    A = rng.standard_normal((3, 1100, 40)).astype(np.float32)
    B = rng.standard_normal((3, 40, 18)).astype(np.float32)
    got = host(functors.gemm(lut, dev(A), dev(B)))
    for i in range(3):
        want = cpu.gemm(img, 11, A[i], B[i])
        assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32))
    got = host(functors.gemm(lut, dev(A), dev(B[1])))
    for i in range(3):
        want = cpu.gemm(img, 11, A[i], B[1])
        assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("kind,m", [("MBM", 11), ("MIT", 8)])
@pytest.mark.parametrize("shape", [((2, 12, 12, 64), (3, 3, 64, 10), (1, 1), "SAME"),    # 576 filter elements: one 1024-row tile
                                   ((1, 9, 10, 128), (3, 3, 128, 20), (1, 1), "VALID"),  # 1152: one 2048-row tile
                                   ((2, 15, 14, 40), (4, 4, 40, 9), (2, 2), "SAME"),     # 640, strided
                                   ((1, 8, 8, 300), (3, 3, 300, 5), (1, 1), "SAME")])    # 2700: 4096-row tile
def test_filter_gradient_on_row_staged_engine(luts, kind, m, shape):
    """Filter gradients with 512 or more filter elements run on the row-staged engine too (rows =
    filter elements, reduction = pixels) when the table-aware query sizes the workspace; with the
    reduction kept whole the result is bit-equal to the oracle's loop nest."""
    from approxtrain_amd import functors
    lut, img = luts(kind, m)
    xs, ws, st, padding = shape
    rng = np.random.default_rng(m * 10 + xs[1] + ws[2])
    x = rng.standard_normal(xs).astype(np.float32)
    x[rng.random(xs) < 0.3] = 0.0
    w = rng.standard_normal(ws).astype(np.float32)
    dy = rng.standard_normal(cpu.conv2d_fwd(img, m, x, w, st, padding).shape).astype(np.float32)
    dw = host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding))
    want = cpu.conv2d_grad_filter(img, m, x, ws, dy, st, padding)
    assert np.array_equal(dw.view(np.uint32), want.view(np.uint32))


def test_sliced_reduction_on_row_staged_engine(luts):
    """With split reductions allowed, a problem of few tiles and a long reduction is cut into slices
    of whole chunks (partial sums added in slice order by the reduction kernel): within
    1e-5 * sum|products| of the sequential oracle, and the same bits run to run; the same call
    through a whole-reduction handle is bit-equal to the oracle."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    whole, img = luts("MBM", 11)
    sliced = ApproxMulLut.from_entries(_legacy(img), 11)
    assert lib.amsim_lut_set_split_k(sliced.handle, 1) == 0
    rng = np.random.default_rng(77)
    # filter gradient: 576 rows x 24 columns, reduction over 4 * 30 * 30 = 3600 pixels (113 chunks)
    xs, ws = (4, 30, 30, 64), (3, 3, 64, 24)
    x = np.maximum(rng.standard_normal(xs), 0).astype(np.float32)
    dy = rng.standard_normal((4, 30, 30, 24)).astype(np.float32)
    want = cpu.conv2d_grad_filter(img, 11, x, ws, dy, (1, 1), "SAME", threads=cpu.max_threads())
    # sum|p| <= exact filter gradient of the absolute values (+ 1 % headroom for the multiplier's error)
    from tests.util import torch_conv_reference
    sum_abs = torch_conv_reference(np.abs(x), np.zeros(ws, np.float32), np.abs(dy), (1, 1), "SAME")[2] * 1.01
    got = host(functors.convam_filter_grad(sliced, dev(x), ws, dev(dy), (1, 1), "SAME"))
    from tests.gpu_util import assert_close_sum_abs
    assert_close_sum_abs(got, want, sum_abs)
    again = host(functors.convam_filter_grad(sliced, dev(x), ws, dev(dy), (1, 1), "SAME"))
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    exact = host(functors.convam_filter_grad(whole, dev(x), ws, dev(dy), (1, 1), "SAME"))
    assert np.array_equal(exact.view(np.uint32), want.view(np.uint32))
    # a dense product of the same kind: 1000 x 16 outputs over a reduction of 6000
    A = rng.standard_normal((1000, 6000)).astype(np.float32)
    B = rng.standard_normal((6000, 16)).astype(np.float32)
    got = host(functors.gemm(sliced, dev(A), dev(B)))
    want = cpu.gemm(img, 11, A, B, threads=cpu.max_threads())
    assert_close_sum_abs(got, want, np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64) * 1.01)


@pytest.mark.parametrize("M,N,K", [(600, 20, 50), (1024, 9, 33), (1500, 40, 70), (2048, 8, 64), (2050, 17, 40)])
def test_row_staged_tile_heights(luts, M, N, K):
    """512..1024 rows run as one 1024-row tile, up to 2048 as one 2048-row tile, more as 4096-row
    (or half-height) tiles: each bit-equal to the oracle."""
    from approxtrain_amd import functors
    lut, img = luts("MIT", 11)
    rng = np.random.default_rng(M + N + K)
    A, B = _ops(rng, M, N, K, 0, 0)
    got = host(functors.gemm(lut, dev(A), dev(B)))
    assert np.array_equal(got.view(np.uint32), cpu.gemm(img, 11, A, B).view(np.uint32))


SPECIALS = np.array([np.inf, -np.inf, np.nan, 1e-40, -1e-42, 3e38, -3e38, 1e-30, 2e-38, 0.0, -0.0], dtype=np.float32)


def _spice(rng, a, p):
    if p <= 0:
        return a
    hit = rng.random(a.shape) < p
    a = a.copy()
    a[hit] = rng.choice(SPECIALS, size=int(hit.sum()))
    return a


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_on_wide_tables(luts, seed):
    """Seeded sweep at shapes that reach the row-staged engine (512 or more rows over the lanes):
    GEMMs with transposes and batches, and the three convolution passes, for widths 8..11; a third of
    the cases carry special values (inf, NaN, subnormals, huge, tiny) in every operand.  Whole
    reductions: bit-equal to the oracle (NaN as a class)."""
    from approxtrain_amd import functors
    rng = np.random.default_rng(4000 + seed)
    m = int(rng.choice([8, 9, 10, 11]))
    kind = str(rng.choice(["MBM", "MIT"]))
    lut, img = luts(kind, m)
    p = (0.0, 0.0, 0.003)[seed % 3]
    if seed % 2 == 0:
        big, small, K = int(rng.integers(512, 5000)), int(rng.integers(1, 40)), int(rng.integers(1, 150))
        M, N = (big, small) if seed % 4 == 0 else (small, big)
        nb = int(rng.choice([0, 0, 2]))
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        sa = ((nb,) if nb else ()) + ((K, M) if ta else (M, K))
        sb = ((nb,) if nb else ()) + ((N, K) if tb else (K, N))
        A = _spice(rng, rng.standard_normal(sa).astype(np.float32), p)
        B = _spice(rng, rng.standard_normal(sb).astype(np.float32), p)
        got = host(functors.gemm(lut, dev(A), dev(B), trans_a=ta, trans_b=tb))
        if nb:
            want = np.stack([cpu.gemm(img, m, A[i], B[i], transA=int(ta), transB=int(tb)) for i in range(nb)])
        else:
            want = cpu.gemm(img, m, A, B, transA=int(ta), transB=int(tb))
        assert got.shape == want.shape and np.all(same_bits_or_both_nan(got, want)), (m, M, N, K, nb, ta, tb)
    else:
        c = int(rng.choice([3, 8, 24, 64, 70]))
        oc = int(rng.choice([1, 5, 16, 24]))
        kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        if kh * kw * c < 512 and seed % 4 == 1:
            c = -(-512 // (kh * kw)) + int(rng.integers(0, 9))      # enough filter elements for the filter gradient's rows
        n, h, w = int(rng.integers(1, 4)), int(rng.integers(kh + 8, kh + 30)), int(rng.integers(kw + 8, kw + 30))
        st = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        padding = str(rng.choice(["SAME", "VALID"]))
        xs, ws = (n, h, w, c), (kh, kw, c, oc)
        x = _spice(rng, rng.standard_normal(xs).astype(np.float32) * (rng.random(xs) > 0.3), p)
        wt = _spice(rng, rng.standard_normal(ws).astype(np.float32), p)
        want_y = cpu.conv2d_fwd(img, m, x, wt, st, padding)
        dy = _spice(rng, rng.standard_normal(want_y.shape).astype(np.float32), p)
        got = [host(functors.convam(lut, dev(x), dev(wt), st, padding)),
               host(functors.convam_input_grad(lut, xs, dev(wt), dev(dy), st, padding)),
               host(functors.convam_filter_grad(lut, dev(x), ws, dev(dy), st, padding))]
        want = [want_y, cpu.conv2d_grad_input(img, m, xs, wt, dy, st, padding),
                cpu.conv2d_grad_filter(img, m, x, ws, dy, st, padding)]
        for g, v in zip(got, want):
            assert np.all(same_bits_or_both_nan(g, v)), (m, xs, ws, st, padding)


@pytest.mark.parametrize("sa,sb", [(-90, 0), (0, -100), (-70, -50), (-100, -40), (60, 30), (100, 30), (-126, 40)])
def test_row_staged_gemm_far_off_exponents(luts, sa, sb):
    """Operands scaled by 2^sa and 2^sb: far outside the quick test's exponent interval, yet most
    pairs of ranges still allow the fast product form (tiny times ordinary); where the products
    would under- or overflow the chunk takes the full-domain product.  Bit-equal either way."""
    from approxtrain_amd import functors
    lut, img = luts("MBM", 11)
    rng = np.random.default_rng(abs(sa) * 7 + abs(sb))
    A, B = _ops(rng, 1100, 24, 70, 0, 0)
    A = (A * np.float32(2.0) ** sa).astype(np.float32)
    B = (B * np.float32(2.0) ** sb).astype(np.float32)
    got = host(functors.gemm(lut, dev(A), dev(B)))
    want = cpu.gemm(img, 11, A, B)
    assert np.all(same_bits_or_both_nan(got, want))
