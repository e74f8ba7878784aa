"""The entry points only enqueue kernels on the caller's stream (no allocation,
no synchronisation, no memset or copy nodes), so a training step can be captured
into a HIP graph and replayed.  Every replay is checked against the eager result
on the same inputs, bit for bit, with eager work and synchronisation between
replays."""
import numpy as np
import pytest
import torch

from tests.gpu_util import host
from tests.util import lut_path

pytestmark = pytest.mark.gpu
MBM = lut_path("MBM", 7)


def _bits(t):
    return host(t).view(np.uint32)


def _step(lut, x, w, dy):
    from approxtrain_amd import functors
    y = functors.convam(lut, x, w, (1, 1), "SAME", bias=None, activation=None)
    dx = functors.convam_input_grad(lut, tuple(x.shape), w, dy, (1, 1), "SAME")
    dw = functors.convam_filter_grad(lut, x, tuple(w.shape), dy, (1, 1), "SAME")   # splits its reduction
    return y, dx, dw


def test_conv_training_step_replays_from_a_graph():
    from approxtrain_amd import ApproxMulLut
    lut = ApproxMulLut.cached(MBM)
    gen = torch.Generator(device="cuda").manual_seed(3)
    shape_x, shape_w, shape_y = (4, 28, 28, 32), (3, 3, 32, 48), (4, 28, 28, 48)
    x, w, dy = (torch.randn(s, device="cuda", generator=gen) for s in (shape_x, shape_w, shape_y))
    _step(lut, x, w, dy)                       # warm-up outside the capture (plans, LUT upload)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _step(lut, x, w, dy)
    for _ in range(3):
        for t in (x, w, dy):                   # new values in the captured input buffers
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        eager = _step(lut, x, w, dy)
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert np.array_equal(_bits(got), _bits(want))


def test_attention_and_dense_replay_from_a_graph():
    from approxtrain_amd import ApproxMulLut, functors
    lut = ApproxMulLut.cached(MBM)
    gen = torch.Generator(device="cuda").manual_seed(4)
    q, k, v, go = (torch.randn(6, 64, 32, device="cuda", generator=gen) for _ in range(4))
    wt = torch.randn(32, 40, device="cuda", generator=gen)
    bias = torch.randn(40, device="cuda", generator=gen)

    def step():
        out, wts = functors.attention(lut, q, k, v, 5.0)
        grads = functors.attention_grad(lut, q, k, v, wts, go, 5.0)
        proj = functors.denseam(lut, out.reshape(-1, 32), wt, bias=bias, activation="relu")
        return (out, wts, proj) + tuple(grads)

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for _ in range(3):
        for t in (q, k, v, go):
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        eager = step()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert np.array_equal(_bits(got), _bits(want))


def test_whole_training_step_with_autograd_and_optimizer_replays_from_a_graph():
    """LeNet-5-shaped model through the layers: forward, loss, autograd backward and the SGD
    update captured as one graph.  The loss of every replay must follow the eager run's
    trajectory (same seeds, same data), step by step."""
    from tests.test_gpu_training import _lenet
    rng = np.random.default_rng(0)
    protos = rng.standard_normal((10, 28, 28, 1)).astype(np.float32)
    labels = rng.integers(0, 10, 128)
    data = protos[labels] + 0.5 * rng.standard_normal((128, 28, 28, 1)).astype(np.float32)
    x, y = torch.from_numpy(data).cuda(), torch.from_numpy(labels).cuda()

    def trajectory(graphed, steps=12):
        torch.manual_seed(0)
        model = _lenet()
        opt = torch.optim.SGD(model.parameters(), lr=0.05, momentum=0.9)

        def step():
            opt.zero_grad(set_to_none=False)
            loss = torch.nn.functional.cross_entropy(model(x), y)
            loss.backward()
            opt.step()
            return loss.detach()

        losses = []
        side = torch.cuda.Stream()                       # warm-up off the default stream, as capture requires
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                losses.append(float(step()))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        if graphed:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_loss = step()
            for _ in range(steps):
                graph.replay()
                torch.cuda.synchronize()
                losses.append(float(static_loss))
        else:
            for _ in range(steps):
                losses.append(float(step()))
        return np.array(losses)

    eager, replayed = trajectory(False), trajectory(True)
    assert np.all(np.isfinite(eager)) and eager[-1] < eager[0]      # it trains
    np.testing.assert_allclose(replayed, eager, rtol=2e-4, atol=1e-6)
