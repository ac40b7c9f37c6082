"""Imperative optimizers with the interface of ``raf.optim.SGD`` and ``raf.optim.LANS``
(python/raf/optim/sgd.py:22-58, python/raf/optim/lans.py:22-103 in the reference), on torch
tensors that live on a ROCm device.  Parameters carry their gradient in ``.grad`` like the
reference's ndarrays do.
"""
from __future__ import annotations

import torch

from . import op as _op


class SGD:
    """Stochastic gradient descent with momentum: one ``raf.op.sgd`` call per parameter."""

    def __init__(self, params, learning_rate, momentum=0):
        if learning_rate < 0.0:
            raise ValueError("Invalid learning rate: {}".format(learning_rate))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        self.params = []
        self._lr = learning_rate
        self._momentum = momentum
        for x in params:
            assert isinstance(x, torch.Tensor), "Only tensors can be optimized!"
            self.params.append((x, torch.zeros_like(x)))  # velocity starts at zero (sgd.py:47-49)

    def step(self):
        """Update the parameters with gradients."""
        for x0, v0 in self.params:
            if x0.grad is None:
                continue
            v1, x1 = _op.sgd(x0.data, x0.grad, v0, self._lr, self._momentum)
            # the reference rebinds the arrays (x0.update(x1)); the same effect on a torch
            # parameter is a device-to-device copy into its storage
            x0.data.copy_(x1)
            v0.copy_(v1)


class LANS:
    """LANS (http://arxiv.org/abs/2006.13484): one multi-tensor ``raf.op.lans`` call per step."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-6, weight_decay=0.01,
                 bias_correction=True, grad_averaging=True, mode=True, normalize_grad=True):
        self.lr = lr
        self.beta1 = betas[0]
        self.beta2 = betas[1]
        self.eps = eps
        self.weight_decay = weight_decay
        self.bias_correction = bias_correction
        self.grad_averaging = grad_averaging
        self.mode = mode
        self.normalize_grad = normalize_grad
        self.params = []
        self._step = 1  # lans.py:66
        for x in params:
            assert isinstance(x, torch.Tensor), "Only tensors can be optimized!"
            self.params.append((x, torch.zeros_like(x), torch.zeros_like(x)))

    def step(self):
        """Update the parameters with gradients."""
        g_list, x_list, m_list, v_list = [], [], [], []
        for x, m, v in self.params:
            if x.grad is None:
                continue
            g_list.append(x.grad)
            x_list.append(x.data)
            m_list.append(m)
            v_list.append(v)
        if not x_list:
            self._step += 1
            return
        step = torch.tensor(float(self._step), dtype=torch.float32, device=x_list[0].device)
        tensor_list = g_list + x_list + m_list + v_list  # lans.py:89
        _op.lans(tensor_list, step, self.lr, self.beta1, self.beta2, self.eps, self.bias_correction,
                 self.weight_decay, self.grad_averaging, self.mode, self.normalize_grad)
        self._step += 1
