"""The reference's optimizer tests train a small convolution / batch-norm / linear classifier and
compare the weights after every step (tests/python/optim/test_sgd.py:83-128 against
torch.optim.SGD at 1e-4; tests/python/optim/test_lans.py:97-137 against apex FusedLANS at 1e-3).
The same loop here: torch supplies the model and its gradients, raf_amd.optim the optimizer step;
SGD is compared with torch.optim.SGD as there, LANS (apex is not installed) with the float64 oracle
fed the same gradients."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import lans_f64
from oracle.lans_f64 import LansHParams

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class SmallClassifier(nn.Module):
    """3-channel image -> 5x5 convolution to 6 channels -> batch norm -> sigmoid -> 2x2 average pool
    -> linear layer -> log-softmax loss (the shape of the reference tests' model)."""

    def __init__(self, side, classes, conv_bias):
        super().__init__()
        self.conv = nn.Conv2d(3, 6, kernel_size=5, padding=2, bias=conv_bias)
        self.norm = nn.BatchNorm2d(6)
        self.head = nn.Linear((side // 2) ** 2 * 6, classes)

    def forward(self, x, target):
        h = torch.sigmoid(self.norm(self.conv(x)))
        h = torch.flatten(F.avg_pool2d(h, (2, 2), (2, 2)), 1)
        return F.nll_loss(F.log_softmax(self.head(h), dim=-1), target)


def _batch(gen, side, classes):
    x = torch.randn(1, 3, side, side, device=DEV, generator=gen)
    y = torch.randint(0, classes, (1,), device=DEV, generator=gen)
    return x, y


def test_sgd_training_follows_torch(native_libs):
    from raf_amd import optim

    torch.manual_seed(0)
    side, classes, steps = 32, 10, 10
    ours = SmallClassifier(side, classes, conv_bias=True).to(DEV).train()
    theirs = copy.deepcopy(ours)
    m_opt = optim.SGD(list(ours.parameters()), 0.1, 0.01)  # test_sgd.py:98
    t_opt = torch.optim.SGD(theirs.parameters(), lr=0.1, momentum=0.01)
    gen = torch.Generator(device=DEV).manual_seed(1)
    for _ in range(steps):
        x, y = _batch(gen, side, classes)
        for model, opt in ((ours, m_opt), (theirs, t_opt)):
            model.zero_grad()
            loss = model(x, y)
            loss.backward()
            opt.step()
        for (name, a), b in zip(ours.named_parameters(), theirs.parameters()):
            np.testing.assert_allclose(a.detach().cpu().numpy(), b.detach().cpu().numpy(), rtol=1e-4, atol=1e-4,
                                       err_msg=name)


def test_lans_training_follows_the_oracle(native_libs):
    from raf_amd import optim

    torch.manual_seed(0)
    side, classes, steps = 32, 10, 4
    model = SmallClassifier(side, classes, conv_bias=False).to(DEV).train()
    params = list(model.parameters())
    m_opt = optim.LANS(params)  # defaults of raf.optim.LANS, python/raf/optim/lans.py:44-55
    ow = [p.detach().cpu().numpy().ravel().copy() for p in params]
    om = [np.zeros_like(a) for a in ow]
    ov = [np.zeros_like(a) for a in ow]
    gen = torch.Generator(device=DEV).manual_seed(2)
    for step in range(1, steps + 1):
        x, y = _batch(gen, side, classes)
        model.zero_grad()
        model(x, y).backward()
        grads = [p.grad.detach().cpu().numpy().ravel().copy() for p in params]
        m_opt.step()
        ow, om, ov, _ = lans_f64.lans_step(grads, ow, om, ov, step, LansHParams())
        for (name, p), want in zip(model.named_parameters(), ow):
            got = p.detach().cpu().numpy().ravel()
            np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-3, err_msg=name)  # the reference's bar
            assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) <= 1e-5 * step, name
        # the next step starts from the model's own weights on both sides: one step at a time is compared
        ow = [p.detach().cpu().numpy().ravel().copy() for p in params]


# ------------------------------------------------------------------ the optimizer objects' own bookkeeping
def _lans_reference(g, w, m, v, step, **kw):
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, step, LansHParams(**kw))
    return ow, om, ov


def test_parameters_without_a_gradient_are_skipped(native_libs):
    """Like the reference (python/raf/optim/lans.py:81-83, sgd.py:53-56): a parameter whose grad is
    None is left out of the step, and joins again once it has one; the state of the others does
    not care."""
    from raf_amd import optim

    rng = np.random.default_rng(7)
    sizes = [1000, 77, 4097, 5]
    init = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
    params = [torch.from_numpy(a.copy()).to(DEV).requires_grad_() for a in init]
    opt = optim.LANS(params)
    for p, g in zip(params, grads):
        p.grad = torch.from_numpy(g).to(DEV)
    params[1].grad = None
    opt.step()  # step 1 without parameter 1
    params[1].grad = torch.from_numpy(grads[1]).to(DEV)
    opt.step()  # step 2 with all four
    torch.cuda.synchronize()
    zeros = [np.zeros_like(a) for a in init]
    live = [0, 2, 3]
    w1, m1, v1 = _lans_reference([grads[i] for i in live], [init[i] for i in live], [zeros[i] for i in live],
                                 [zeros[i] for i in live], 1)
    w, m, v = list(init), list(zeros), list(zeros)
    for j, i in enumerate(live):
        w[i], m[i], v[i] = w1[j], m1[j], v1[j]
    w2, _, _ = _lans_reference(grads, w, m, v, 2)
    for p, want in zip(params, w2):
        got = p.detach().cpu().numpy()
        assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-12)) <= 1e-5

    sgd_params = [torch.from_numpy(a.copy()).to(DEV).requires_grad_() for a in init]
    sgd = optim.SGD(sgd_params, 0.1, 0.9)
    for p, g in zip(sgd_params, grads):
        p.grad = torch.from_numpy(g).to(DEV)
    sgd_params[2].grad = None
    sgd.step()
    torch.cuda.synchronize()
    assert np.array_equal(sgd_params[2].detach().cpu().numpy(), init[2])
    assert not np.array_equal(sgd_params[0].detach().cpu().numpy(), init[0])


def test_half_precision_model_whose_storage_is_replaced(native_libs):
    """The optimizer keeps aliases of the half-precision parameters' data between steps; a parameter
    whose storage has been swapped (x.data = ...) must receive the next weights in its new storage."""
    from raf_amd import optim

    torch.manual_seed(3)
    params = [torch.randn(n, device=DEV).mul_(0.02).half().requires_grad_() for n in (3000, 17, 9000)]
    opt = optim.LANS(params)
    for p in params:
        p.grad = (torch.randn(p.shape, device=DEV) * 1e-3).half()
    opt.step()
    old_storage = params[1].data
    before = old_storage.clone()
    params[1].data = params[1].data.clone()  # same values, new storage
    opt.step()
    torch.cuda.synchronize()
    assert torch.equal(old_storage, before)  # the old storage is no longer written
    master = opt.params[1][1]
    assert torch.equal(params[1].data, master.half())  # the new one holds the narrowed master weight
    assert not torch.equal(params[1].data, before)


def test_optimizer_step_replayed_from_a_hip_graph(native_libs):
    """A model of many small tensors is host-bound in eager mode (one attribute read and one address
    check per tensor and step); captured once, `LANS.step()` replays with no Python at all and gives
    the eager results."""
    from raf_amd import optim, shapes

    sizes = shapes.log_uniform_numels(300, seed=21)
    torch.manual_seed(5)
    init = [torch.randn(n, device=DEV).mul_(0.02) for n in sizes]
    grads = [torch.randn(n, device=DEV).mul_(1e-3) for n in sizes]

    def fresh():
        ps = [t.clone().requires_grad_() for t in init]
        for p, g in zip(ps, grads):
            p.grad = g.clone()
        return ps, optim.LANS(ps)

    eager_params, eager = fresh()
    for _ in range(6):
        eager.step()
    params, opt = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up: plan, tables and workspace exist before the capture
        opt.step()
        opt.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        opt.step()  # step 3 is recorded, not run
    for _ in range(4):  # replays: steps 3 to 6 (the step counter lives on the device)
        graph.replay()
    torch.cuda.synchronize()
    for a, b in zip(params, eager_params):
        assert torch.equal(a.detach(), b.detach())
