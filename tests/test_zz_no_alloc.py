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
