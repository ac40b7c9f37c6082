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
