"""LUT-multiply GEMM, dense and matmul entry points on the GPU (through the C
ABI) against the CPU oracle on the same seeded inputs.

Bars: with the reduction unsplit every output is one ascending-k FP32 chain,
so results are BIT-EQUAL to the oracle; with split-K (small problems) they are
within 1e-5 * sum_k |product| (the tolerance the task states)."""
import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, asym_lut_u8, dev, host, lut32
from tests.util import lut_path, small_ints

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("amsim_engine")]


@pytest.fixture(scope="module")
def amd():
    import approxtrain_amd
    from approxtrain_amd import functors
    lib = approxtrain_amd.load_library()
    yield functors
    lib.amsim_set_split_k(1)


def _set_split(mode):
    import approxtrain_amd
    approxtrain_amd.load_library().amsim_set_split_k(mode)


def _ops(rng, M, N, K, ta, tb, relu=False):
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    if relu:
        A = np.maximum(A, 0)
    return A, B


@pytest.mark.parametrize("M,N,K", [(64, 16, 32), (100, 37, 77), (257, 300, 129), (1, 1, 1), (3, 130, 40),
                                   (130, 3, 40), (65, 6, 150), (200, 1, 33), (128, 300, 784)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_bit_equal_when_unsplit(amd, M, N, K, ta, tb):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    rng = np.random.default_rng(M * 7 + N * 3 + K + ta * 2 + tb)
    A, B = _ops(rng, M, N, K, ta, tb, relu=True)
    lut = ApproxMulLut(lut_path("MBM", 7))
    got = host(amd.gemm(lut, dev(A), dev(B), trans_a=bool(ta), trans_b=bool(tb)))
    want = cpu.gemm(lut32("MBM", 7), 7, A, B, transA=ta, transB=tb)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("kind,m", [("MBM", 1), ("MBM", 3), ("MBM", 5), ("MIT", 1), ("MIT", 3), ("MIT", 5),
                                    ("MIT", 7), ("ACC", 7)])
def test_gemm_every_lut_width(amd, kind, m):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    rng = np.random.default_rng(50 + m)
    A, B = _ops(rng, 150, 70, 96, 0, 0)
    got = host(amd.gemm(ApproxMulLut(lut_path(kind, m)), dev(A), dev(B)))
    want = cpu.gemm(lut32(kind, m), m, A, B)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("swap", [False, True])
@pytest.mark.parametrize("M,N", [(90, 20), (20, 90)])  # both lane orientations
def test_gemm_operand_order_with_asymmetric_lut(amd, swap, M, N):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    tab = asym_lut_u8(3)
    lut = ApproxMulLut.from_entries(tab, 3)
    rng = np.random.default_rng(61)
    A, B = _ops(rng, M, N, 45, 0, 0)
    got = host(amd.gemm(lut, dev(A), dev(B), swap_operands=swap))
    want = cpu.gemm(cpu.expand_u8(tab, 3), 3, A, B, swap=swap)
    other = cpu.gemm(cpu.expand_u8(tab, 3), 3, A, B, swap=not swap)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert not np.array_equal(want, other)


def test_gemm_full_domain_operands_take_exact_path(amd):
    """Subnormals, infinities, NaNs, huge and tiny magnitudes inside the
    operands: the flagged chunks must reproduce the functional-model product."""
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    rng = np.random.default_rng(62)
    M, N, K = 96, 40, 128
    A = (rng.standard_normal((M, K)) * 2.0 ** rng.integers(-70, 70, (M, K))).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 2.0 ** rng.integers(-70, 70, (K, N))).astype(np.float32)
    A[3, 5] = np.float32(1e-41); A[10, 40] = np.inf; A[20, 70] = np.nan; A[0, 0] = 0.0; A[50, 100] = -0.0
    B[5, 3] = np.float32(-3e-40); B[64, 7] = -np.inf; B[33, 1] = np.float32(3e38); B[100, 2] = 0.0
    got = host(amd.gemm(ApproxMulLut(lut_path("MBM", 7)), dev(A), dev(B)))
    with np.errstate(all="ignore"):
        want = cpu.gemm(lut32("MBM", 7), 7, A, B)
    both_nan = np.isnan(got) & np.isnan(want)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | both_nan).all()
    assert np.isnan(want).any() and np.isinf(want).any()


def test_gemm_split_k_within_tolerance_and_deterministic(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(1)
    rng = np.random.default_rng(63)
    A, B = _ops(rng, 128, 300, 784, 0, 0)
    lut = ApproxMulLut(lut_path("MBM", 7))
    got = host(amd.gemm(lut, dev(A), dev(B)))
    again = host(amd.gemm(lut, dev(A), dev(B)))
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    want = cpu.gemm(lut32("MBM", 7), 7, A, B)
    assert_close_sum_abs(got, want, cpu.gemm_abs(lut32("MBM", 7), 7, A, B))


def test_gemm_exact_on_integers(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(1)
    rng = np.random.default_rng(64)
    A, B = small_ints(rng, (200, 333)), small_ints(rng, (333, 50))
    got = host(amd.gemm(ApproxMulLut(lut_path("ACC", 7)), dev(A), dev(B)))
    assert np.array_equal(got.astype(np.int64), A.astype(np.int64) @ B.astype(np.int64))


def test_gemm_strided_batch_and_broadcast(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    rng = np.random.default_rng(65)
    lut = ApproxMulLut(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    A = rng.standard_normal((5, 70, 48)).astype(np.float32)
    B = rng.standard_normal((5, 48, 33)).astype(np.float32)
    got = host(amd.gemm(lut, dev(A), dev(B)))
    for i in range(5):
        assert np.array_equal(got[i].view(np.uint32), cpu.gemm(L, 7, A[i], B[i]).view(np.uint32))
    got = host(amd.gemm(lut, dev(A), dev(B[0])))
    for i in range(5):
        assert np.array_equal(got[i].view(np.uint32), cpu.gemm(L, 7, A[i], B[0]).view(np.uint32))
    got = host(amd.gemm(lut, dev(A[0]), dev(B), trans_b=False))
    for i in range(5):
        assert np.array_equal(got[i].view(np.uint32), cpu.gemm(L, 7, A[0], B[i]).view(np.uint32))


@pytest.mark.parametrize("ba,bb", [(0, 0), (3, 3), (3, 1), (1, 3), (3, 0), (0, 3)])
def test_matmulam_shape_cases(amd, ba, bb):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    rng = np.random.default_rng(66)
    a = rng.standard_normal(((ba,) if ba else ()) + (40, 24)).astype(np.float32)
    b = rng.standard_normal(((bb,) if bb else ()) + (24, 50)).astype(np.float32)
    got = host(amd.matmulam(ApproxMulLut(lut_path("MIT", 7)), dev(a), dev(b)))
    want = cpu.matmul(lut32("MIT", 7), 7, a, b)
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_matmulam_errors_and_empty(amd):
    from approxtrain_amd import AmsimError, ApproxMulLut
    lut = ApproxMulLut(lut_path("MIT", 7))
    with pytest.raises(AmsimError):
        amd.matmulam(lut, torch.zeros(2, 3, device="cuda"), torch.zeros(4, 5, device="cuda"))
    with pytest.raises(AmsimError):
        amd.matmulam(lut, torch.zeros(2, 2, 3, device="cuda"), torch.zeros(3, 3, 5, device="cuda"))
    out = amd.matmulam(lut, torch.zeros(4, 0, device="cuda"), torch.zeros(0, 5, device="cuda"))
    assert out.shape == (4, 5) and float(out.abs().sum()) == 0.0  # matmulam.cc:154-160
    out = amd.matmulam(lut, torch.zeros(0, 3, device="cuda"), torch.zeros(3, 5, device="cuda"))
    assert out.shape == (0, 5)


def test_denseam_lenet300_first_layer(amd):
    """denseam forward at LeNet-300-100's first layer: X[128,784] uniform[0,1),
    W[784,300] Glorot-uniform, MBM_7; plus both gradients."""
    from approxtrain_amd import ApproxMulLut
    lut = ApproxMulLut(lut_path("MBM", 7))
    L = lut32("MBM", 7)
    x = np.random.default_rng(1).random((128, 784), dtype=np.float32)
    lim = np.sqrt(6.0 / (784 + 300))
    w = np.random.default_rng(2).uniform(-lim, lim, (784, 300)).astype(np.float32)
    dy = (np.random.default_rng(3).standard_normal((128, 300)) * 0.1).astype(np.float32)
    _set_split(0)
    y = host(amd.denseam(lut, dev(x), dev(w)))
    assert np.array_equal(y.view(np.uint32), cpu.dense_fwd(L, 7, x, w).view(np.uint32))
    dx, dw = amd.denseam_grad(lut, dev(dy), dev(x), dev(w))
    dx_ref, dw_ref = cpu.dense_grad(L, 7, dy, x, w)
    assert np.array_equal(host(dx).view(np.uint32), dx_ref.view(np.uint32))
    assert np.array_equal(host(dw).view(np.uint32), dw_ref.view(np.uint32))
    _set_split(1)
    y = host(amd.denseam(lut, dev(x), dev(w)))
    assert_close_sum_abs(y, cpu.dense_fwd(L, 7, x, w), cpu.gemm_abs(L, 7, x, w))


def test_dense_grad_operand_order(amd):
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    tab = asym_lut_u8(3)
    lut = ApproxMulLut.from_entries(tab, 3)
    rng = np.random.default_rng(67)
    x, w, dy = (rng.standard_normal(s).astype(np.float32) for s in ((30, 50), (50, 40), (30, 40)))
    dx, dw = amd.denseam_grad(lut, dev(dy), dev(x), dev(w))
    dx_ref, dw_ref = cpu.dense_grad(cpu.expand_u8(tab, 3), 3, dy, x, w)
    assert np.array_equal(host(dx).view(np.uint32), dx_ref.view(np.uint32))
    assert np.array_equal(host(dw).view(np.uint32), dw_ref.view(np.uint32))


@pytest.mark.parametrize("kind", ["MBM", "MIT"])
@pytest.mark.parametrize("m", [9, 11])
def test_gemm_wide_mantissa_lut_gathered_from_global_memory(amd, kind, m):
    """Mantissa widths above 7 (the 2^22-entry m = 11 table does not fit the
    LDS): 32-bit legacy entries in, LUT gathered through L2.  No reference
    file or model exists for these widths; the table comes from the oracle's
    generator (closed-form rules that reproduce every m <= 7 file)."""
    from approxtrain_amd import ApproxMulLut
    _set_split(0)
    img = cpu.lutgen32(kind, m)
    legacy = (((img >> 23) << 31) | (img & 0x7fffff)).astype(np.uint32)
    lut = ApproxMulLut.from_entries(legacy, m)
    rng = np.random.default_rng(80 + m)
    for (M, N, K, ta, tb) in [(130, 70, 96, 0, 0), (64, 16, 40, 1, 0), (20, 200, 64, 0, 1)]:
        A, B = _ops(rng, M, N, K, ta, tb)
        A[0, 0] = np.float32(1e-40)  # one flagged chunk takes the exact path
        got = host(amd.gemm(lut, dev(A), dev(B), trans_a=bool(ta), trans_b=bool(tb)))
        want = cpu.gemm(img, m, A, B, transA=ta, transB=tb)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_generated_table_files_load_and_multiply(amd, tmp_path):
    """Tables written by the generation tool (1-byte entries at width 5, 4-byte entries at
    width 9) go through amsim_lut_load_file and give the oracle's GEMM bit for bit."""
    from approxtrain_amd import ApproxMulLut, lut_gen
    _set_split(0)
    rng = np.random.default_rng(91)
    for kind, m in (("MIT", 5), ("MBM", 9)):
        entries = lut_gen.generate_builtin(kind, m, lut_gen.file_entry_bytes(m))
        lut = ApproxMulLut(lut_gen.write_table(entries, kind, m, str(tmp_path)))
        assert lut.mant_width == m
        A, B = _ops(rng, 70, 40, 64, 0, 0)
        got = host(amd.gemm(lut, dev(A), dev(B)))
        want = cpu.gemm(cpu.lutgen32(kind, m), m, A, B)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _plan(M, N, K, batch=1, ta=0, tb=0):
    import ctypes as C
    import approxtrain_amd
    info = (C.c_int64 * 8)()
    assert approxtrain_amd.load_library().amsim_gemm_plan_info(ta, tb, M, N, K, batch, info) == 0
    return dict(zip(("TN", "WR", "nsplit", "cps", "rows_main", "tail_nsplit", "tail_cps", "chunks"), info))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,expect", [
    (100352, 64, 576, "tail"),          # one round and a bit: unsplit main part + split tail
    (25088, 128, 1152, "split+tail"),   # half a round: main part split in two, tail split further
    (6272, 256, 2304, "split+tail"),
    (512, 512, 8192, "split"),          # few outputs, long reduction
    (51200, 64, 128, "whole"),          # short reduction: nothing to gain from splitting
    (40, 6, 50000, "slices+split"),     # one row tile: all four waves on its one column group
    (200704, 1, 150, "tail"),           # 256-row workgroups (one narrow column group): 768 slots + a split tail
    (50176, 6, 400, "split"),           # 256-row workgroups, reduction split three ways
    (2048, 1024, 256, "slices+tail"),   # few row tiles, short reduction: its rows dealt out to a workgroup's four waves
    (2048, 256, 1024, "slices+split"),  # ... and split across workgroups as well
    (8192, 128, 256, "slices"),
])
def test_planner_paths_match_the_oracle(amd, M, N, K, expect):
    """The work-shaping decisions (reduction split, tail rows split further, both with partial sums)
    at shapes that take each path: result within 1e-5 * sum|products| of the sequential oracle."""
    from approxtrain_amd import ApproxMulLut
    p = _plan(M, N, K)
    split, tail = p["nsplit"] > 1, p["tail_nsplit"] > 0
    assert (p["WR"] == 0) == expect.startswith("slices"), p
    assert {"tail": (not split) and tail, "split+tail": split and tail, "split": split and not tail,
            "whole": (not split) and (not tail), "slices": (not split) and (not tail), "slices+split": split and not tail,
            "slices+tail": (not split) and tail}[expect], p
    _set_split(1)
    rng = np.random.default_rng(M + N + K)
    # a sample of the rows keeps the oracle fast: the GPU computes everything, rows are independent
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    lut = ApproxMulLut.cached(lut_path("MBM", 7))
    got = host(amd.gemm(lut, dev(A), dev(B)))
    rows = np.unique(np.concatenate([np.arange(min(M, 70)), rng.integers(0, M, 60), np.arange(max(M - 300, 0), M)]))
    L = lut32("MBM", 7)
    want = cpu.gemm(L, 7, A[rows].copy(), B)
    assert_close_sum_abs(got[rows], want, cpu.gemm_abs(L, 7, A[rows].copy(), B), 1e-5)


def test_gemm_one_term_reductions_cover_every_operand_pattern_width7(amd):
    """K = 1 makes every output a single product that went through the GEMM kernel's own product
    form (LUT byte + exponent bits as one FMA factor on the fast path, the full-domain product in
    flagged chunks): all 2^16 x 2^16 pairs of (sign, exponent, 7-bit mantissa) operand patterns
    must equal 0 + the oracle's LUT product, bit for bit (NaNs as a class)."""
    from concurrent.futures import ThreadPoolExecutor
    from approxtrain_amd import ApproxMulLut
    from tests.util import lut_bytes, same_bits_or_both_nan
    _set_split(0)
    lut = ApproxMulLut(lut_path("MBM", 7))
    L = cpu.expand_u8(lut_bytes("MBM", 7), 7)
    n, block = 1 << 16, 1 << 11
    pats = (np.arange(n, dtype=np.uint32) << 16)
    A = torch.from_numpy(pats.view(np.float32).reshape(n, 1).copy()).cuda()
    workers = min(16, cpu.max_threads())
    a_host = pats.view(np.float32)
    bad = total = 0
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for j0 in range(0, n, block):
            b_host = pats[j0:j0 + block].view(np.float32)
            got = host(amd.gemm(lut, A, torch.from_numpy(b_host.reshape(1, block).copy()).cuda()))   # [n, block]

            def rows(r):
                a = np.repeat(a_host[r[0]:r[-1] + 1], block)
                b = np.tile(b_host, r.size)
                with np.errstate(invalid="ignore"):
                    want = cpu.lut_mul_array(L, 7, a, b) + np.float32(0.0)  # the accumulator starts at +0
                return int((~same_bits_or_both_nan(got[r[0]:r[-1] + 1].ravel(), want)).sum())

            bad += sum(pool.map(rows, np.array_split(np.arange(n), workers * 2)))
            total += n * block
    assert total == 1 << 32 and bad == 0, f"{bad} of {total} one-term outputs differ"
