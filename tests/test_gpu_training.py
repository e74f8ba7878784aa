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
