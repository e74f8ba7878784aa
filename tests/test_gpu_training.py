"""End to end through the layers: a LeNet-5-shaped network (the reference's mnist_example.py
model: AMConv2D 5x5 x6 SAME -> pool -> AMConv2D 5x5 x16 VALID -> pool -> denseam 120 -> 84 -> 10)
with the MBM_7 multiplier learns a synthetic 10-class problem; every multiplication of
activations by weights, forward and backward, goes through the approximate GEMM."""
import numpy as np
import pytest
import torch

from tests.util import lut_path

pytestmark = pytest.mark.gpu
MBM = lut_path("MBM", 7)


def _lenet():
    from approxtrain_amd.layers import AMConv2D, denseam

    class LeNet(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.c1 = AMConv2D(6, 5, padding="same", activation="relu", mant_mul_lut=MBM, in_channels=1)
            self.c2 = AMConv2D(16, 5, padding="valid", activation="relu", mant_mul_lut=MBM, in_channels=6)
            self.d1 = denseam(120, activation="relu", mant_mul_lut=MBM, input_dim=400)
            self.d2 = denseam(84, activation="relu", mant_mul_lut=MBM, input_dim=120)
            self.d3 = denseam(10, mant_mul_lut=MBM, input_dim=84)

        def forward(self, x):  # NHWC
            pool = lambda t: torch.nn.functional.avg_pool2d(t.permute(0, 3, 1, 2), 2).permute(0, 2, 3, 1).contiguous()
            x = pool(self.c1(x))
            x = pool(self.c2(x))
            return self.d3(self.d2(self.d1(x.reshape(x.shape[0], -1))))

    return LeNet().cuda()


def test_lenet_learns_a_synthetic_problem():
    torch.manual_seed(0)
    rng = np.random.default_rng(0)
    # ten class prototypes + noise, 28 x 28 x 1
    protos = rng.standard_normal((10, 28, 28, 1)).astype(np.float32)
    labels = rng.integers(0, 10, 256)
    data = protos[labels] + 0.5 * rng.standard_normal((256, 28, 28, 1)).astype(np.float32)
    x, y = torch.from_numpy(data).cuda(), torch.from_numpy(labels).cuda()
    model = _lenet()
    opt = torch.optim.SGD(model.parameters(), lr=0.05, momentum=0.9)
    losses = []
    for step in range(40):
        opt.zero_grad()
        loss = torch.nn.functional.cross_entropy(model(x), y)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(np.isfinite(losses))
    assert losses[-1] < 0.5 * losses[0], losses
    with torch.no_grad():
        acc = float((model(x).argmax(1) == y).float().mean())
    assert acc > 0.8, acc
    # every parameter received a gradient through the approximate ops
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


def test_resnet_bottleneck_block_runs_through_the_library():
    """A ResNet-50 bottleneck (1x1 reduce -> 3x3 -> 1x1 expand, identity shortcut, stride-2 variant
    with a projection shortcut): every convolution, forward and backward, is an AMConv2D.  Each
    layer's output is checked against the oracle on that layer's actual input, and the block's
    parameters all receive finite gradients."""
    import approxtrain_amd
    from approxtrain_amd.layers import AMConv2D
    from oracle import cpu
    from tests.gpu_util import host, lut32
    lib = approxtrain_amd.load_library()
    L = lut32("MBM", 7)

    class Bottleneck(torch.nn.Module):
        def __init__(self, cin, mid, cout, stride):
            super().__init__()
            conv = lambda f, k, s, a, c: AMConv2D(f, k, strides=s, padding="same", activation=a, mant_mul_lut=MBM, in_channels=c)
            self.a = conv(mid, 1, 1, "relu", cin)
            self.b = conv(mid, 3, stride, "relu", mid)
            self.c = conv(cout, 1, 1, None, mid)
            self.proj = conv(cout, 1, stride, None, cin) if (stride != 1 or cin != cout) else None

        def forward(self, x):
            self.seen = [x]
            h = self.a(x); self.seen.append(h)
            h = self.b(h); self.seen.append(h)
            h = self.c(h); self.seen.append(h)
            short = x if self.proj is None else self.proj(x)
            return torch.relu(h + short)

    torch.manual_seed(1)
    lib.amsim_set_split_k(0)
    try:
        for cin, mid, cout, stride, hw in ((64, 16, 64, 1, 14), (64, 32, 128, 2, 14)):
            block = Bottleneck(cin, mid, cout, stride).cuda()
            x = torch.randn(2, hw, hw, cin, device="cuda", requires_grad=True)
            y = block(x)
            assert tuple(y.shape) == (2, hw // stride, hw // stride, cout)
            for layer, xin, out in zip((block.a, block.b, block.c), block.seen[:-1], block.seen[1:]):
                want = cpu.conv2d_fwd(L, 7, host(xin), host(layer.kernel), tuple(layer.strides), "SAME") + host(layer.bias)
                if layer.activation is not None:
                    want = np.where(want < 0, np.float32(0), want)
                assert np.array_equal(host(out).view(np.uint32), want.astype(np.float32).view(np.uint32))
            y.square().mean().backward()
            assert torch.isfinite(x.grad).all() and float(x.grad.abs().sum()) > 0
            assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in block.parameters())
    finally:
        lib.amsim_set_split_k(1)
