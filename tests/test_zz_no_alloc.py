"""The allocation-free forward convolution (amsim_convam_noalloc_f32) against the entry point it
is a variant of (amsim_convam_f32 with a caller's workspace), through the C ABI: same inputs,
same plan, so the outputs must be bit-identical.  Two calls in a row share the library's one
scratch buffer on the GPU; the second is smaller, so stale contents of the first would show."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.gpu_util import dev, host
from tests.util import lut_path

pytestmark = pytest.mark.gpu


def _both(lib, lut, x, w, padding):
    from approxtrain_amd import functors
    from approxtrain_amd._lib import check, conv_geometry
    n, h, wd, c = x.shape
    kh, kw, _, oc = w.shape
    oh, pt = conv_geometry(h, kh, 1, padding)
    ow, pl = conv_geometry(wd, kw, 1, padding)
    xd, wdv = dev(x), dev(w)
    want = host(functors.convam(lut, xd, wdv, (1, 1), padding))
    out = torch.full((n, oh, ow, oc), float("nan"), dtype=torch.float32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    check(lib.amsim_convam_noalloc_f32(lut.handle, C.c_void_p(xd.data_ptr()), C.c_void_p(out.data_ptr()), n, oh, ow, oc,
                                       1, 1, pl, pt, kh, kw, c, wd, h, C.c_void_p(wdv.data_ptr()), stream))
    torch.cuda.synchronize()
    return host(out), want


def test_noalloc_convolution_matches_workspace_entry_point_twice_in_a_row():
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut(lut_path("MBM", 7))
    rng = np.random.default_rng(77)
    # first call: a split tail (1568 row tiles on 1536 slots) -> partial sums in the scratch
    x1 = np.maximum(rng.standard_normal((32, 56, 56, 64)), 0).astype(np.float32)
    w1 = (rng.standard_normal((3, 3, 64, 64)) * 0.06).astype(np.float32)
    got, want = _both(lib, lut, x1, w1, "SAME")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # second call, smaller, other shape: split reduction over few outputs
    x2 = rng.standard_normal((2, 9, 11, 24)).astype(np.float32)
    w2 = rng.standard_normal((3, 2, 24, 10)).astype(np.float32)
    got, want = _both(lib, lut, x2, w2, "VALID")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and the first again: the buffer is reusable in any order
    got, want = _both(lib, lut, x1, w1, "SAME")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _noalloc_call(lib, lut, xd, wdv, out, padding, stream):
    from approxtrain_amd._lib import check, conv_geometry
    n, h, wd, c = xd.shape
    kh, kw, _, oc = wdv.shape
    oh, pt = conv_geometry(h, kh, 1, padding)
    ow, pl = conv_geometry(wd, kw, 1, padding)
    check(lib.amsim_convam_noalloc_f32(lut.handle, C.c_void_p(xd.data_ptr()), C.c_void_p(out.data_ptr()), n, oh, ow, oc,
                                       1, 1, pl, pt, kh, kw, c, wd, h, C.c_void_p(wdv.data_ptr()), C.c_void_p(stream)))


def test_noalloc_convolution_under_graph_capture():
    """After one warm-up call (the first call on a device looks the scratch array's address up), the
    entry point is captured into a HIP graph -- capture fails on any allocation or synchronisation,
    so this also shows that the call makes none -- and replayed on new inputs: every replay equals
    the workspace entry point bit for bit."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut(lut_path("MBM", 7))
    rng = np.random.default_rng(78)
    xs, ws = (8, 28, 28, 32), (3, 3, 32, 48)
    xd = dev(np.maximum(rng.standard_normal(xs), 0).astype(np.float32))
    wdv = dev((rng.standard_normal(ws) * 0.1).astype(np.float32))
    out = torch.full((8, 28, 28, 48), float("nan"), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _noalloc_call(lib, lut, xd, wdv, out, "SAME", side.cuda_stream)  # warm-up, outside the capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            _noalloc_call(lib, lut, xd, wdv, out, "SAME", torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for seed in (1, 2, 3):
        r = np.random.default_rng(seed)
        xd.copy_(dev(np.maximum(r.standard_normal(xs), 0).astype(np.float32)))
        wdv.copy_(dev((r.standard_normal(ws) * 0.1).astype(np.float32)))
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = host(functors.convam(lut, xd, wdv, (1, 1), "SAME"))
        assert np.array_equal(host(out).view(np.uint32), want.view(np.uint32)), seed


def test_noalloc_convolution_with_a_wide_table_matches_the_same_scratch_size():
    """Tables of 8..11 mantissa bits pick their engine by the scratch they are given, so the
    guarantee is stated against amsim_convam_f32 with a workspace of AMSIM_NOALLOC_SCRATCH_BYTES."""
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    from approxtrain_amd._lib import check, conv_geometry
    from oracle import cpu
    lib = approxtrain_amd.load_library()
    L = cpu.lutgen32("MBM", 11)
    lut = ApproxMulLut.from_entries((((L >> 23) << 31) | (L & 0x7fffff)).astype(np.uint32), 11)
    rng = np.random.default_rng(79)
    x = np.maximum(rng.standard_normal((2, 16, 16, 16)), 0).astype(np.float32)
    w = (rng.standard_normal((3, 3, 16, 32)) * 0.1).astype(np.float32)
    xd, wdv = dev(x), dev(w)
    out = torch.full((2, 16, 16, 32), float("nan"), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _noalloc_call(lib, lut, xd, wdv, out, "SAME", stream)
    scratch_bytes = 32 << 20
    ws = torch.empty(scratch_bytes + 256, dtype=torch.uint8, device="cuda")
    wsp = ws.data_ptr() + (-ws.data_ptr()) % 256
    want = torch.full_like(out, float("nan"))
    oh, pt = conv_geometry(16, 3, 1, "SAME")
    ow, pl = conv_geometry(16, 3, 1, "SAME")
    check(lib.amsim_convam_f32(lut.handle, C.c_void_p(xd.data_ptr()), C.c_void_p(want.data_ptr()), 2, oh, ow, 32, 1, 1, pl, pt,
                               3, 3, 16, 16, 16, C.c_void_p(wdv.data_ptr()), C.c_void_p(wsp), scratch_bytes, C.c_void_p(stream)))
    torch.cuda.synchronize()
    assert np.array_equal(host(out).view(np.uint32), host(want).view(np.uint32))
    # and both are the oracle's sequential chains when the handle keeps reductions whole
    assert lib.amsim_lut_set_split_k(lut.handle, 0) == 0
    _noalloc_call(lib, lut, xd, wdv, out, "SAME", stream)
    torch.cuda.synchronize()
    ref = cpu.conv2d_fwd(L, 11, x, w, (1, 1), "SAME", threads=8)
    assert np.array_equal(host(out).view(np.uint32), ref.view(np.uint32))


def test_noalloc_convolution_refuses_what_does_not_fit():
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut
    lib = approxtrain_amd.load_library()
    lut = ApproxMulLut(lut_path("MBM", 7))
    # 7x7x512 -> 1024 filter: 25 088 x 1024 pre-decoded words alone exceed the 32 MiB scratch
    n, h, wd, c, kh, kw, oc = 1, 8, 8, 512, 7, 7, 1024
    assert lib.amsim_convam_workspace_bytes(n, h, wd, oc, kh, kw, c) > (32 << 20)
    x = torch.zeros((n, h, wd, c), device="cuda")
    w = torch.zeros((kh, kw, c, oc), device="cuda")
    out = torch.zeros((n, h, wd, oc), device="cuda")
    rc = lib.amsim_convam_noalloc_f32(lut.handle, C.c_void_p(x.data_ptr()), C.c_void_p(out.data_ptr()), n, h, wd, oc, 1, 1,
                                      3, 3, kh, kw, c, wd, h, C.c_void_p(w.data_ptr()), None)
    assert rc == 6 and b"allocation-free" in lib.amsim_last_error()
