"""Thin Python handles over the C ABI, operating on torch tensors that live on a ROCm device.

torch is only the owner of device memory and of the current HIP stream here; every computation is
done by the HIP kernels behind ``include/rafhip_optim.h``.
"""
from __future__ import annotations

import ctypes
from ctypes import c_double, c_float, c_int64, c_void_p
from typing import List, Optional, Sequence

import torch

from . import _lib
from ._lib import LansHParams, RAFHIP_BF16, RAFHIP_F16, RAFHIP_F32, RAFHIP_F64, check


def _current_stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_gpu_f32(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name}: expected a tensor on the GPU, got device {t.device}")
    if t.dtype != torch.float32:
        raise TypeError(f"{name}: expected float32, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")


def sgd_f32(x: torch.Tensor, dx: torch.Tensor, v: torch.Tensor, learning_rate: float, mu: float,
            v_out: Optional[torch.Tensor] = None, x_out: Optional[torch.Tensor] = None):
    """``rafhip_sgd_f32`` on torch tensors; returns ``(v1, x1)`` (new tensors unless given)."""
    for t, name in ((x, "x"), (dx, "dx"), (v, "v")):
        _require_gpu_f32(t, name)
    if not (x.shape == dx.shape == v.shape):
        raise ValueError(f"sgd: shapes differ: x{tuple(x.shape)} dx{tuple(dx.shape)} v{tuple(v.shape)}")
    v1 = torch.empty_like(dx) if v_out is None else v_out
    x1 = torch.empty_like(dx) if x_out is None else x_out
    check(_lib.optim().rafhip_sgd_f32(x.data_ptr(), dx.data_ptr(), v.data_ptr(), v1.data_ptr(),
                                      x1.data_ptr(), x.numel(), float(learning_rate), float(mu),
                                      _current_stream(x.device)))
    return v1, x1


_DTYPE_CODE = {torch.float32: RAFHIP_F32, torch.float16: RAFHIP_F16, torch.bfloat16: RAFHIP_BF16}


def sgd(x: torch.Tensor, dx: torch.Tensor, v: torch.Tensor, learning_rate: float, mu: float):
    """``rafhip_sgd``: the step in the tensors' own element type (float32, float64, float16 or
    bfloat16, the same for all three); returns new ``(v1, x1)``."""
    code = {**_DTYPE_CODE, torch.float64: _lib.RAFHIP_F64}.get(x.dtype)
    if code is None or dx.dtype != x.dtype or v.dtype != x.dtype:
        raise TypeError("sgd: x, dx and v must share one of float32, float64, float16, bfloat16")
    for t, name in ((x, "x"), (dx, "dx"), (v, "v")):
        if not t.is_cuda or not t.is_contiguous():
            raise TypeError(f"sgd: {name} must be a contiguous GPU tensor")
    if not (x.shape == dx.shape == v.shape):
        raise ValueError(f"sgd: shapes differ: x{tuple(x.shape)} dx{tuple(dx.shape)} v{tuple(v.shape)}")
    v1, x1 = torch.empty_like(dx), torch.empty_like(dx)
    check(_lib.optim().rafhip_sgd(x.data_ptr(), dx.data_ptr(), v.data_ptr(), v1.data_ptr(), x1.data_ptr(),
                                  x.numel(), code, float(learning_rate), float(mu), _current_stream(x.device)))
    return v1, x1


class SgdPlan:
    """Owns a ``rafhip_sgd_plan``: momentum SGD over a whole parameter list, in place, one launch."""

    def __init__(self, numels: Sequence[int], grad_dtype=torch.float32, device="cuda:0"):
        self._h = c_void_p(None)
        self.lib = _lib.optim()
        self.device = torch.device(device)
        self.numels = [int(n) for n in numels]
        self.n = len(self.numels)
        if grad_dtype not in _DTYPE_CODE:
            raise TypeError(f"SGD gradients must be float32, float16 or bfloat16, got {grad_dtype}")
        self.grad_dtype = grad_dtype
        arr = (c_int64 * max(self.n, 1))(*self.numels)
        with torch.cuda.device(self.device):
            check(self.lib.rafhip_sgd_plan_create(self.n, arr, _DTYPE_CODE[grad_dtype], ctypes.byref(self._h)))

    def close(self):
        if self._h:
            self.lib.rafhip_sgd_plan_destroy(self._h)
            self._h = c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def _ptrs(self, tensors, dtype, what, optional=False):
        if len(tensors) != self.n:
            raise ValueError(f"{what}: expected {self.n} tensors, got {len(tensors)}")
        arr = (c_void_p * max(self.n, 1))()
        for i, t in enumerate(tensors):
            if t is None and optional:
                continue
            if not t.is_cuda or t.dtype != dtype or not t.is_contiguous() or t.numel() != self.numels[i]:
                raise TypeError(f"{what}[{i}]: need a contiguous {dtype} GPU tensor of {self.numels[i]} elements")
            arr[i] = t.data_ptr()
        return arr

    def marshal(self, x, dx, v, p=None):
        """Pointer lists for ``step``; reusable while the tensors stay where they are."""
        pp, p_code = None, RAFHIP_F16
        if p is not None:
            dt = next((t.dtype for t in p if t is not None), torch.float16)
            if dt not in (torch.float16, torch.bfloat16):
                raise TypeError(f"16-bit weight copies must be float16 or bfloat16, got {dt}")
            pp, p_code = self._ptrs(p, dt, "p", optional=True), _DTYPE_CODE[dt]
        return (self._ptrs(x, torch.float32, "x"), self._ptrs(dx, self.grad_dtype, "dx"),
                self._ptrs(v, torch.float32, "v"), pp, p_code, (list(x), list(dx), list(v), p))

    def step(self, x, dx, v, learning_rate: float, mu: float, p=None, marshalled=None):
        """x, v updated in place; ``p``: optional float16 / bfloat16 tensors receiving the new x."""
        xp, dp, vp, pp, p_code, _ = marshalled if marshalled is not None else self.marshal(x, dx, v, p)
        check(self.lib.rafhip_sgd_multi_step(self._h, xp, dp, vp, pp, p_code, float(learning_rate),
                                             float(mu), _current_stream(self.device)))


_NORM_DTYPES = {torch.float32: RAFHIP_F32, torch.float64: RAFHIP_F64, torch.float16: RAFHIP_F16,
                torch.bfloat16: RAFHIP_BF16}


def l2norm(x: torch.Tensor, out: Optional[torch.Tensor] = None,
           workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``rafhip_l2norm``: sqrt(sum x^2) as a 0-d tensor of x's dtype, left on the device."""
    if not x.is_cuda or not x.is_contiguous():
        raise ValueError("l2norm: expected a contiguous tensor on the GPU")
    if x.dtype not in _NORM_DTYPES:
        raise TypeError(f"l2norm: unsupported dtype {x.dtype}")
    lib = _lib.optim()
    if out is None:
        out = torch.empty((), dtype=x.dtype, device=x.device)
    elif out.dtype != x.dtype or out.numel() != 1 or not out.is_cuda:
        raise TypeError("l2norm: out must be a one-element GPU tensor of x's dtype")
    need = lib.rafhip_l2norm_workspace_bytes(x.numel())
    if workspace is None and need > 0:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    check(lib.rafhip_l2norm(x.data_ptr(), _NORM_DTYPES[x.dtype], x.numel(), out.data_ptr(),
                            workspace.data_ptr() if workspace is not None else None,
                            workspace.numel() if workspace is not None else 0,
                            _current_stream(x.device)))
    return out


class FusePlan:
    """Owns a ``rafhip_fuse_plan`` for a list of tensors of fixed byte sizes: ``fuse`` packs them
    back to back into one flat buffer, ``defuse`` unpacks it, one kernel launch each."""

    def __init__(self, nbytes: Sequence[int], device="cuda:0"):
        self._h = c_void_p(None)
        self.lib = _lib.optim()
        self.device = torch.device(device)
        self.nbytes = [int(b) for b in nbytes]
        self.n = len(self.nbytes)
        arr = (c_int64 * max(self.n, 1))(*self.nbytes)
        with torch.cuda.device(self.device):
            check(self.lib.rafhip_fuse_plan_create(self.n, arr, ctypes.byref(self._h)))
        self.total_bytes = self.lib.rafhip_fuse_plan_total_bytes(self._h)

    def close(self):
        if self._h:
            self.lib.rafhip_fuse_plan_destroy(self._h)
            self._h = c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def _ptrs(self, parts: Sequence[torch.Tensor]):
        if len(parts) != self.n:
            raise ValueError(f"expected {self.n} tensors, got {len(parts)}")
        arr = (c_void_p * max(self.n, 1))()
        for i, t in enumerate(parts):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"parts[{i}]: need a contiguous GPU tensor")
            if t.numel() * t.element_size() != self.nbytes[i]:
                raise ValueError(f"parts[{i}]: {t.numel() * t.element_size()} bytes, plan has {self.nbytes[i]}")
            arr[i] = t.data_ptr()
        return arr

    def _check_flat(self, flat: torch.Tensor):
        if not flat.is_cuda or not flat.is_contiguous() or flat.numel() * flat.element_size() != self.total_bytes:
            raise ValueError(f"flat buffer: need a contiguous GPU tensor of {self.total_bytes} bytes")

    def fuse(self, parts: Sequence[torch.Tensor], flat: torch.Tensor) -> torch.Tensor:
        self._check_flat(flat)
        check(self.lib.rafhip_fuse_tensors(self._h, self._ptrs(parts), flat.data_ptr(),
                                           _current_stream(self.device)))
        return flat

    def defuse(self, flat: torch.Tensor, parts: Sequence[torch.Tensor]):
        self._check_flat(flat)
        check(self.lib.rafhip_defuse_tensor(self._h, flat.data_ptr(), self._ptrs(parts),
                                            _current_stream(self.device)))
        return parts


def make_hparams(learning_rate=1e-3, beta1=0.9, beta2=0.999, eps=1e-6, bias_correction=1,
                 weight_decay=0.01, grad_averaging=1, mode=1, normalize_grad=True,
                 grad_unscale=1.0) -> LansHParams:
    """Python numbers -> the fp32/int schema fields (bools become 0/1 like the reference's FFI)."""
    return LansHParams(float(learning_rate), float(beta1), float(beta2), float(eps),
                       int(bias_correction), float(weight_decay), int(grad_averaging), int(mode),
                       int(bool(normalize_grad)), float(grad_unscale))


def query_layout(numels: Sequence[int]):
    """(n_chunks, workspace_bytes) for a tensor list; host arithmetic only, needs no GPU."""
    n = len(numels)
    arr = (c_int64 * max(n, 1))(*numels)
    chunks, ws = c_int64(0), c_int64(0)
    check(_lib.optim().rafhip_lans_query_layout(n, arr, ctypes.byref(chunks), ctypes.byref(ws)))
    return chunks.value, ws.value


def pipeline_order(numels: Sequence[int], group_elements: int = 0, **options):
    """[(pass, tensor, chunk)] in the order the pipelined schedule hands out work; host arithmetic.
    ``options``: fields of ``rafhip_lans_plan_options`` that cut the list (``round_slices``,
    ``stream_from_elements``, ``stream_hold_items``)."""
    n = len(numels)
    arr = (c_int64 * max(n, 1))(*numels)
    count = c_int64(0)
    lib = _lib.optim()
    if not options:
        order = lambda buf, cap: lib.rafhip_lans_pipeline_order(n, arr, group_elements, buf, cap, ctypes.byref(count))
    else:
        o = _lib.LansPlanOptions.defaults(**options)
        if group_elements > 0:
            o.group_elements = group_elements
        order = lambda buf, cap: lib.rafhip_lans_pipeline_order_with(n, arr, ctypes.byref(o), buf, cap,
                                                                     ctypes.byref(count))
    check(order(None, 0))
    buf = (ctypes.c_int32 * max(3 * count.value, 1))()
    check(order(buf, count.value))
    return [(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(count.value)]


class LansPlan:
    """Owns a ``rafhip_lans_plan`` and a workspace tensor sized for it."""

    def __init__(self, numels: Sequence[int], grad_dtype=torch.float32, device="cuda:0", **options):
        """``options``: fields of ``rafhip_lans_plan_options`` (``schedule``, ``group_elements``,
        ``round_slices``, ``blocks_per_cu``, ``stream_from_elements``, ``stream_hold_items``,
        ``resident_mib``, ``apply_slice_shift``, ``spin_limit``); none changes a result."""
        self._h = c_void_p(None)
        self.lib = _lib.optim()
        self.device = torch.device(device)
        self.numels = [int(n) for n in numels]
        self.n = len(self.numels)
        if grad_dtype not in _DTYPE_CODE:
            raise TypeError(f"LANS gradients must be float32, float16 or bfloat16, got {grad_dtype}")
        code = _DTYPE_CODE[grad_dtype]
        self.grad_dtype = grad_dtype
        arr = (c_int64 * max(self.n, 1))(*self.numels)
        with torch.cuda.device(self.device):
            if options:
                o = _lib.LansPlanOptions.defaults(**options)
                check(self.lib.rafhip_lans_plan_create_with(self.n, arr, code, ctypes.byref(o), ctypes.byref(self._h)))
            else:
                check(self.lib.rafhip_lans_plan_create(self.n, arr, code, ctypes.byref(self._h)))
        self.workspace_bytes = self.lib.rafhip_lans_workspace_bytes(self._h)
        self.n_chunks = self.lib.rafhip_lans_plan_num_chunks(self._h)
        self.total_elements = self.lib.rafhip_lans_plan_total_elements(self._h)
        self.workspace = torch.empty(max(self.workspace_bytes, 256), dtype=torch.uint8,
                                     device=self.device)

    def set_schedule(self, schedule: str):
        """"phased" (one launch per pass) or "pipelined" (one persistent, cache-aware launch)."""
        code = {"phased": _lib.RAFHIP_LANS_PHASED, "pipelined": _lib.RAFHIP_LANS_PIPELINED}[schedule]
        check(self.lib.rafhip_lans_plan_set_schedule(self._h, code))

    @property
    def schedule(self) -> str:
        return {0: "phased", 1: "pipelined"}[self.lib.rafhip_lans_plan_schedule(self._h)]

    @property
    def table_uploads(self) -> int:
        """How often a pointer table had to be sent to the device so far."""
        return self.lib.rafhip_lans_plan_table_uploads(self._h)

    def close(self):
        if self._h:
            self.lib.rafhip_lans_plan_destroy(self._h)
            self._h = c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def _ptrs(self, tensors: Sequence[torch.Tensor], dtype, what: str):
        if len(tensors) != self.n:
            raise ValueError(f"{what}: expected {self.n} tensors, got {len(tensors)}")
        arr = (c_void_p * max(self.n, 1))()
        for i, t in enumerate(tensors):
            if not t.is_cuda or t.dtype != dtype or not t.is_contiguous():
                raise TypeError(f"{what}[{i}]: need a contiguous {dtype} GPU tensor, "
                                f"got {t.dtype} on {t.device}")
            if t.numel() != self.numels[i]:
                raise ValueError(f"{what}[{i}]: {t.numel()} elements, plan has {self.numels[i]}")
            arr[i] = t.data_ptr()
        return arr

    def _model_ptrs(self, p):
        """Pointer list and dtype code of the optional 16-bit weight copies."""
        if p is None:
            return None, RAFHIP_F16
        dt = next((t.dtype for t in p if t is not None), torch.float16)
        if dt not in (torch.float16, torch.bfloat16):
            raise TypeError(f"16-bit weight copies must be float16 or bfloat16, got {dt}")
        if len(p) != self.n:
            raise ValueError(f"p: expected {self.n} tensors, got {len(p)}")
        arr = (c_void_p * max(self.n, 1))()
        for i, t in enumerate(p):
            if t is None:
                continue
            if not t.is_cuda or t.dtype != dt or not t.is_contiguous() or t.numel() != self.numels[i]:
                raise TypeError(f"p[{i}]: need a contiguous {dt} GPU tensor of {self.numels[i]} elements")
            arr[i] = t.data_ptr()
        return arr, _DTYPE_CODE[dt]

    def step(self, g: Sequence[torch.Tensor], w: Sequence[torch.Tensor],
             m: Sequence[torch.Tensor], v: Sequence[torch.Tensor], step, hp: LansHParams,
             workspace: Optional[torch.Tensor] = None, p: Optional[Sequence] = None):
        """``step`` is a 0-d fp32 GPU tensor (read on the device) or a Python int.  ``p``: optional
        float16 / bfloat16 tensors (entries may be None) that receive the new weights narrowed to
        16 bits: the half-precision model parameters of a mixed-precision run."""
        ws = self.workspace if workspace is None else workspace
        pp, p_code = self._model_ptrs(p)
        gp = self._ptrs(g, self.grad_dtype, "g")
        wp = self._ptrs(w, torch.float32, "w")
        mp = self._ptrs(m, torch.float32, "m")
        vp = self._ptrs(v, torch.float32, "v")
        if isinstance(step, torch.Tensor):
            if step.dtype != torch.float32 or step.numel() != 1 or not step.is_cuda:
                raise TypeError("step tensor must be a 0-d float32 GPU tensor")
            step_dev, step_host = step.data_ptr(), 0
        else:
            step_dev, step_host = None, int(step)
        check(self.lib.rafhip_lans_step_mixed(self._h, gp, wp, mp, vp, pp, p_code, step_dev, step_host,
                                              ctypes.byref(hp), ws.data_ptr(), ws.numel(),
                                              _current_stream(self.device)))

    def step_noalloc(self, g, w, m, v, step, hp: LansHParams, p: Optional[Sequence] = None):
        """``rafhip_lans_step_noalloc``: the same step on the library's static scratch array instead
        of a workspace; no device memory is allocated by the call."""
        pp, p_code = self._model_ptrs(p)
        gp = self._ptrs(g, self.grad_dtype, "g")
        wp = self._ptrs(w, torch.float32, "w")
        mp = self._ptrs(m, torch.float32, "m")
        vp = self._ptrs(v, torch.float32, "v")
        if isinstance(step, torch.Tensor):
            if step.dtype != torch.float32 or step.numel() != 1 or not step.is_cuda:
                raise TypeError("step tensor must be a 0-d float32 GPU tensor")
            step_dev, step_host = step.data_ptr(), 0
        else:
            step_dev, step_host = None, int(step)
        check(self.lib.rafhip_lans_step_noalloc(self._h, gp, wp, mp, vp, pp, p_code, step_dev, step_host,
                                                ctypes.byref(hp), _current_stream(self.device)))

    def bind(self, g, w, m, v, hp: LansHParams, workspace: Optional[torch.Tensor] = None, p=None):
        """``rafhip_lans_plan_bind``: check the pointer lists and build the tensor table once for
        tensors that stay where they are; ``step_bound`` then costs one foreign call per step that
        touches no list (a training loop updates the same buffers every step)."""
        ws = self.workspace if workspace is None else workspace
        pp, p_code = self._model_ptrs(p)
        check(self.lib.rafhip_lans_plan_bind(self._h, self._ptrs(g, self.grad_dtype, "g"),
                                             self._ptrs(w, torch.float32, "w"), self._ptrs(m, torch.float32, "m"),
                                             self._ptrs(v, torch.float32, "v"), pp, p_code))
        self._bound = (hp, ws, (list(g), list(w), list(m), list(v), p))

    def step_bound(self, step: torch.Tensor):
        """One step on the tensors given to ``bind``; ``step`` is the 0-d fp32 GPU step tensor."""
        hp, ws, _ = self._bound
        check(self.lib.rafhip_lans_step_bound(self._h, step.data_ptr(), 0, ctypes.byref(hp), ws.data_ptr(),
                                              ws.numel(), _current_stream(self.device)))

    def set_dynamic_scale(self, grad_unscale: Optional[torch.Tensor] = None,
                          found_inf: Optional[torch.Tensor] = None):
        """``rafhip_lans_plan_set_dynamic_scale``: 0-d fp32 GPU tensors holding the reciprocal of the
        loss scale and the overflow flag (non-zero: the step does nothing), read by the kernels."""
        for t, name in ((grad_unscale, "grad_unscale"), (found_inf, "found_inf")):
            if t is not None and (t.dtype != torch.float32 or t.numel() != 1 or not t.is_cuda):
                raise TypeError(f"{name} must be a one-element float32 GPU tensor")
        self._dynamic = (grad_unscale, found_inf)  # keep them alive
        check(self.lib.rafhip_lans_plan_set_dynamic_scale(
            self._h, grad_unscale.data_ptr() if grad_unscale is not None else None,
            found_inf.data_ptr() if found_inf is not None else None))

    def read_norms(self, workspace: Optional[torch.Tensor] = None):
        """[n, 4] float64: ||g||, ||w||, ||u_m||, ||u_g|| of the last step."""
        import numpy as np

        ws = self.workspace if workspace is None else workspace
        out = (c_double * max(4 * self.n, 1))()
        check(self.lib.rafhip_lans_read_norms(self._h, ws.data_ptr(), out,
                                              _current_stream(self.device)))
        return np.array(out[:4 * self.n], dtype=np.float64).reshape(self.n, 4)

    def debug_trace(self):
        """[n_items, 4] uint64 (drawn, unblocked, finished, workgroup) of the last pipelined step, or
        None unless the process runs with RAFHIP_LANS_TRACE=1."""
        import numpy as np

        n = c_int64(0)
        check(self.lib.rafhip_lans_debug_trace(self._h, None, 0, ctypes.byref(n)))
        if n.value == 0:
            return None
        buf = np.zeros((n.value, 4), dtype=np.uint64)
        check(self.lib.rafhip_lans_debug_trace(
            self._h, buf.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)), n.value, ctypes.byref(n)))
        return buf

    def timing_enable(self, slots: int):
        check(self.lib.rafhip_lans_timing_enable(self._h, int(slots)))

    def timing_read(self, slot: int) -> List[float]:
        out = (c_float * 5)()
        check(self.lib.rafhip_lans_timing_read(self._h, int(slot), out))
        return list(out)
