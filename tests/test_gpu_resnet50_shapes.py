"""Every convolution shape the benchmark times for ResNet-50 (both layer lists of bench.py: feature
maps 56 -> 7 and the CIFAR-sized 32 -> 4), at the benchmark's batch of 32 -- the work planner's
decisions (reduction splits, tails, reduction slices inside a workgroup, residue classes of strided
gradients) depend on the row count, so smaller look-alikes would exercise other code paths.

Per layer, through the C ABI: forward and grad-input of the full batch, images 0 and 31 recomputed by
the CPU oracle; grad-filter against the oracle on a 2-image slice and, at full batch, through
additivity over the batch.  Default mode: within 1e-5 * sum|products| (the task's bar); with the
handle's reductions kept whole (amsim_lut_set_split_k(h, 0)) the sampled images and the 2-image
filter gradient are bit-equal to the oracle's sequential chains."""
import math
import os
import sys

import numpy as np
import pytest
import torch

from oracle import cpu
from tests.gpu_util import assert_close_sum_abs, host, lut32
from tests.util import lut_path, torch_conv_reference

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402  (the layer lists are the benchmark's own)

pytestmark = pytest.mark.gpu
REL = 1e-5
BATCH = 32
THREADS = 16

LAYERS = [(label,) + tuple(layer[:6]) for label, hw0, cin0 in bench.RESNET50_SIZES for layer in bench.resnet50_layers(hw0, cin0)]


def same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


def filter_grad_abs_bound(x, dy, ws, stride, padding):
    """sum over the batch and pixels of |x| * |dy| per filter element, FP32 on the host (the
    normaliser of the additivity check only)."""
    import torch.nn.functional as F
    from tests.util import tf_same_pads
    xt = torch.from_numpy(np.abs(x)).permute(0, 3, 1, 2).contiguous()
    gt = torch.from_numpy(np.abs(dy)).permute(0, 3, 1, 2).contiguous()
    if padding == "SAME":
        _, pt, pb = tf_same_pads(x.shape[1], ws[0], stride)
        _, pl, pr = tf_same_pads(x.shape[2], ws[1], stride)
        xt = F.pad(xt, (pl, pr, pt, pb))
    w = torch.nn.grad.conv2d_weight(xt, (ws[3], ws[2], ws[0], ws[1]), gt, stride=stride)
    return w.permute(2, 3, 1, 0).numpy().astype(np.float64)


@pytest.mark.parametrize("label,name,hw,cin,cout,k,stride", LAYERS, ids=["%s-%s" % (l[0].split("_")[2], l[1]) for l in LAYERS])
def test_resnet50_layer_at_batch_32(label, name, hw, cin, cout, k, stride):
    from approxtrain_amd import ApproxMulLut, functors
    lib_lut = ApproxMulLut.cached(lut_path("MBM", 7))
    whole = ApproxMulLut(lut_path("MBM", 7))  # a handle of its own whose reductions stay whole
    import approxtrain_amd
    assert approxtrain_amd.load_library().amsim_lut_set_split_k(whole.handle, 0) == 0
    L = lut32("MBM", 7)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1000 + hw * 7 + cin + 3 * cout + k + stride)
    xs, ws, padding, st = (BATCH, hw, hw, cin), (k, k, cin, cout), ("SAME" if k == 3 else "VALID"), (stride, stride)
    xd = torch.relu(torch.randn(*xs, device="cuda", generator=gen))
    wd = torch.randn(*ws, device="cuda", generator=gen) * math.sqrt(2.0 / (k * k * cin))
    y = functors.convam(lib_lut, xd, wd, st, padding)
    dyd = torch.randn(*y.shape, device="cuda", generator=gen)
    dx = functors.convam_input_grad(lib_lut, xs, wd, dyd, st, padding)
    y_whole = functors.convam(whole, xd, wd, st, padding)
    dx_whole = functors.convam_input_grad(whole, xs, wd, dyd, st, padding)
    w = host(wd)
    for img in (0, BATCH - 1):
        xi, dyi = host(xd[img:img + 1]), host(dyd[img:img + 1])
        y_ref = cpu.conv2d_fwd(L, 7, xi, w, st, padding, threads=THREADS)
        dx_ref = cpu.conv2d_grad_input(L, 7, xi.shape, w, dyi, st, padding, threads=THREADS)
        s_y, s_dx, _ = torch_conv_reference(np.abs(xi), np.abs(w), np.abs(dyi), st, padding)
        assert_close_sum_abs(host(y[img:img + 1]), y_ref, s_y, REL)
        assert_close_sum_abs(host(dx[img:img + 1]), dx_ref, s_dx, REL)
        assert same_bits(host(y_whole[img:img + 1]), y_ref), "forward, whole reductions"
        assert same_bits(host(dx_whole[img:img + 1]), dx_ref), "grad-input, whole reductions"
    # filter gradient: two images against the oracle ...
    x2, dy2 = host(xd[:2]), host(dyd[:2])
    dw_ref = cpu.conv2d_grad_filter(L, 7, x2, ws, dy2, st, padding, threads=THREADS)
    _, _, s_dw = torch_conv_reference(np.abs(x2), np.abs(w), np.abs(dy2), st, padding)
    assert_close_sum_abs(host(functors.convam_filter_grad(lib_lut, xd[:2], ws, dyd[:2], st, padding)), dw_ref, s_dw, REL)
    assert same_bits(host(functors.convam_filter_grad(whole, xd[:2], ws, dyd[:2], st, padding)), dw_ref), "grad-filter, whole reductions"
    # ... and the full batch (the plan the benchmark times) through additivity over the batch
    full = host(functors.convam_filter_grad(lib_lut, xd, ws, dyd, st, padding)).astype(np.float64)
    parts = sum(host(functors.convam_filter_grad(lib_lut, xd[i:i + 8], ws, dyd[i:i + 8], st, padding)).astype(np.float64)
                for i in range(0, BATCH, 8))
    assert_close_sum_abs(full, parts, filter_grad_abs_bound(host(xd), host(dyd), ws, stride, padding), REL)
    whole.close()
