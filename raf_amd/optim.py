"""Imperative optimizers with the interface of ``raf.optim.SGD`` and ``raf.optim.LANS``
(python/raf/optim/sgd.py:22-58, python/raf/optim/lans.py:22-103 in the reference), on torch
tensors that live on a ROCm device.  Parameters carry their gradient in ``.grad`` like the
reference's ndarrays do.
"""
from __future__ import annotations

import torch

from . import _lib
from . import op as _op


class SGD:
    """Stochastic gradient descent with momentum.

    ``multi_tensor=False`` follows the reference's imperative optimizer literally: one
    ``raf.op.sgd`` call per parameter and a rebinding of the results (python/raf/optim/sgd.py:51-58).
    The default updates the whole parameter list in place with one multi-tensor launch -- the same
    four roundings per element, so the same bits -- and, for float16 / bfloat16 parameters, keeps
    fp32 master weights and velocities the way the traced optimizer does (sgd.py:152-166,
    :187-215)."""

    def __init__(self, params, learning_rate, momentum=0, multi_tensor=True):
        if learning_rate < 0.0:
            raise ValueError("Invalid learning rate: {}".format(learning_rate))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        self.params = []
        self._lists = None  # the weight and velocity lists of all parameters, made on first use
        self._xs = None  # the parameters themselves as a list, made on first use
        self._model = None  # (data pointers, aliases of the half-precision parameters' data)
        self._lr = learning_rate
        self._momentum = momentum
        params = list(params)
        halves = {x.dtype for x in params if isinstance(x, torch.Tensor)} & {torch.float16, torch.bfloat16}
        self.mixed = bool(halves)
        if self.mixed and (len(halves) > 1 or any(x.dtype not in halves for x in params)):
            raise TypeError("a half-precision model must use one 16-bit dtype for all parameters")
        self.multi_tensor = bool(multi_tensor) or self.mixed
        for x in params:
            assert isinstance(x, torch.Tensor), "Only tensors can be optimized!"
            w = x.data.float() if self.mixed else x.data  # fp32 master weight (sgd.py:152-160)
            self.params.append((x, w, torch.zeros_like(w)))  # velocity starts at zero (sgd.py:47-49)

    def step(self):
        """Update the parameters with gradients."""
        if self._xs is None:
            self._xs = [x for x, _, _ in self.params]
        grads, missing = _lib.glue().grads(self._xs)  # one pass at C speed
        if missing == len(grads):
            return
        live = self.params if not missing else [t for t, g in zip(self.params, grads) if g is not None]
        if not self.multi_tensor:
            for x0, _, v0 in live:
                v1, x1 = _op.sgd(x0.data, x0.grad, v0, self._lr, self._momentum)
                # the reference rebinds the arrays (x0.update(x1)); the same effect on a torch
                # parameter is a device-to-device copy into its storage
                x0.data.copy_(x1)
                v0.copy_(v1)
            return
        if not missing:
            # every parameter has a gradient: the weight and velocity lists made once
            if self._lists is None:
                self._lists = ([w for _, w, _ in self.params], [v for _, _, v in self.params])
            ws, vs = self._lists
        else:
            ws, vs = [w for _, w, _ in live], [v for _, _, v in live]
            grads = [g for g in grads if g is not None]
        tensor_list = ws + grads + vs
        if self.mixed:
            _op.sgd_multi_mixed(tensor_list + self._model_data(live), self._lr, self._momentum)
        else:
            _op.sgd_multi(tensor_list, self._lr, self._momentum)

    def _model_data(self, live):
        """Aliases of the half-precision parameters' data, kept while the storages stay the same."""
        xs = [x for x, _, _ in live]
        ptrs = list(map(torch.Tensor.data_ptr, xs))
        if self._model is None or self._model[0] != ptrs:
            self._model = (ptrs, [x.data for x in xs])
        return self._model[1]


class LANS:
    """LANS (http://arxiv.org/abs/2006.13484): one multi-tensor ``raf.op.lans`` call per step.

    float16 / bfloat16 parameters are trained the way the reference's traced optimizer trains
    them (python/raf/optim/lans.py:213-227, :261-305): an fp32 master copy of every weight holds
    the state, the half gradients feed the op directly and the parameter receives the new master
    weight narrowed to its dtype -- here in one ``lans_mixed`` call instead of
    ``group_cast`` + ``lans`` + ``cast`` + ``add(out=p)``."""

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
        # The step also lives on the device and is advanced there, like the traced optimizer's
        # `step` array (lans.py:228, :240): making a fresh device scalar from the host every step
        # would block on the previous step's kernels.
        self._step_dev = None
        self._lists = None  # the w, m, v lists of all parameters, made on first use
        self._xs = None  # the parameters themselves as a list, made on first use
        self._model = None  # (data pointers, aliases of the half-precision parameters' data)
        params = list(params)
        halves = {x.dtype for x in params if isinstance(x, torch.Tensor)} & {torch.float16, torch.bfloat16}
        self.mixed = bool(halves)
        if self.mixed and (len(halves) > 1 or any(x.dtype not in halves for x in params)):
            raise TypeError("a half-precision model must use one 16-bit dtype for all parameters")
        for x in params:
            assert isinstance(x, torch.Tensor), "Only tensors can be optimized!"
            # the fp32 master weight: the parameter itself, or its widened copy (lans.py:217-219)
            w = x.data.float() if self.mixed else x.data
            self.params.append((x, w, torch.zeros_like(w), torch.zeros_like(w)))

    def step(self):
        """Update the parameters with gradients."""
        params = self.params
        if self._xs is None:
            self._xs = [t[0] for t in params]
        grads, missing = _lib.glue().grads(self._xs)  # one pass at C speed
        if missing:  # the reference skips parameters without a gradient (lans.py:81-83)
            live = [i for i, g in enumerate(grads) if g is not None]
            g_list = [grads[i] for i in live]
            x_list = [params[i][1] for i in live]
            m_list = [params[i][2] for i in live]
            v_list = [params[i][3] for i in live]
            p_list = [params[i][0].data for i in live] if self.mixed else []
        else:
            # The common case costs one attribute read per parameter: the state lists are the ones
            # made at construction, and so are the aliases of the half-precision parameters' data
            # (new ones only if a parameter's storage has been replaced since).
            g_list = grads
            x_list, m_list, v_list = self._state_lists()
            p_list = self._model_data() if self.mixed else []
        if not x_list:
            self._advance()
            return
        if self._step_dev is None or self._step_dev.device != x_list[0].device:
            self._step_dev = torch.tensor(float(self._step), dtype=torch.float32, device=x_list[0].device)
        step = self._step_dev
        tensor_list = g_list + x_list + m_list + v_list  # lans.py:89
        hyper = (self.lr, self.beta1, self.beta2, self.eps, self.bias_correction, self.weight_decay,
                 self.grad_averaging, self.mode, self.normalize_grad)
        if self.mixed:
            _op.lans_mixed(tensor_list + p_list, step, *hyper)
        else:
            _op.lans(tensor_list, step, *hyper)
        self._advance()

    def _state_lists(self):
        if self._lists is None:
            self._lists = tuple([t[i] for t in self.params] for i in (1, 2, 3))
        return self._lists

    def _model_data(self):
        xs = [t[0] for t in self.params]
        ptrs = list(map(torch.Tensor.data_ptr, xs))
        if self._model is None or self._model[0] != ptrs:
            self._model = (ptrs, [x.data for x in xs])
        return self._model[1]

    def _advance(self):
        """``_step`` counts the calls made; the counter the kernels read lives on the device and
        counts the steps that were applied: with dynamic loss scaling in force
        (``op.set_lans_dynamic_scale(found_inf=...)``) a step the kernels skipped because of an
        overflow leaves it where it was, so the bias corrections stay in step with m and v."""
        self._step += 1
        if self._step_dev is not None:
            found_inf = _op.get_lans_dynamic_scale()[1]
            if found_inf is None:
                self._step_dev.add_(1.0)
            else:
                self._step_dev.add_((found_inf == 0).to(torch.float32).reshape(()))
