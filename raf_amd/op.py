"""Imperative operator entry points with the signatures of the reference's generated
``raf._op.imp.sgd`` / ``raf._op.imp.lans`` (argument lists: scripts/src_codegen/def_schema.py:671-694).

Each call walks the same route as in RAF: arguments -> schema -> declare -> dialect dispatch ->
``OpEnv`` -> ``Execute`` (src/impl/interpreter.cc:247-344), implemented by the C++ host layer in
``libraf_hip_dialect.so``; the selected backend is the ``hip`` dialect, whose OpEnvs call the
gfx950 kernels through the C ABI.  OpEnvs are cached per argument signature the way the VM caches
them per (function, pc, shape key) (src/impl/vm/vm.cc:1053-1097).  Tensors are torch tensors on a
ROCm device; torch supplies memory (including the per-call workspace, its caching allocator
standing in for RAF's memory pool) and the current stream, nothing else.
"""
from __future__ import annotations

import collections
import ctypes
from ctypes import c_int64, c_void_p
from typing import Dict, List, Sequence, Tuple

import torch

from . import _lib, runtime
from ._lib import TensorDesc, check_raf

DEV_CPU, DEV_CUDA, DEV_ROCM = 1, 2, 10  # include/raf/device.h:37-50

_DTYPES = {
    torch.float32: (2, 32), torch.float16: (2, 16), torch.float64: (2, 64),
    torch.bfloat16: (4, 16), torch.int32: (0, 32), torch.int64: (0, 64), torch.uint8: (1, 8),
    torch.int8: (0, 8), torch.int16: (0, 16),
}


_SHAPE_ARRAYS = [c_int64 * max(d, 1) for d in range(9)]  # ctypes array types are costly to make


def _desc(t: torch.Tensor, keep: list) -> TensorDesc:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"expected a tensor, got {type(t).__name__}")
    if not t.is_contiguous():
        raise ValueError("tensors must be contiguous")
    code, bits = _DTYPES[t.dtype]
    nd = t.dim()
    shape = (_SHAPE_ARRAYS[nd] if nd < 9 else c_int64 * nd)(*t.shape)
    keep.append(shape)
    # torch on ROCm reports its devices as "cuda"; they are ROCm devices for RAF's purposes.
    dev_type = DEV_ROCM if t.is_cuda else DEV_CPU
    dev_id = t.device.index if t.is_cuda and t.device.index is not None else 0
    return TensorDesc(t.data_ptr(), dev_type, dev_id, code, bits, t.dim(),
                      ctypes.cast(shape, ctypes.POINTER(c_int64)))


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream if t.is_cuda else None


class _Env:
    def __init__(self, handle):
        self.handle = handle
        lib = _lib.dialect()
        self.name = lib.rafhip_raf_env_name(handle).decode()
        self.op = lib.rafhip_raf_env_op(handle).decode()
        self.workspace_bytes = lib.rafhip_raf_env_workspace_bytes(handle)
        self.workspaces = {}  # stream handle -> runtime.Memory
        self.learning_rate = None  # what the OpEnv was made with or last told, if it has one
        self.grad_unscale = 1.0
        self.dynamic_scale = (None, None)  # the tensors the OpEnv was last told to read

    def set_learning_rate(self, learning_rate: float) -> None:
        """A learning-rate schedule keeps its OpEnv: the hip optimizer OpEnvs take a new value between
        two executions (a hip-dialect extension; the reference would build a new OpEnv)."""
        if learning_rate != self.learning_rate:
            check_raf(_lib.dialect().rafhip_raf_env_set_learning_rate(self.handle, learning_rate))
            self.learning_rate = learning_rate

    def set_grad_scaling(self, factor: float, dynamic) -> None:
        """Loss scaling is no part of what identifies an OpEnv either (hip-dialect extension)."""
        if factor != self.grad_unscale:
            check_raf(_lib.dialect().rafhip_raf_env_set_grad_unscale(self.handle, factor))
            self.grad_unscale = factor
        if dynamic[0] is not self.dynamic_scale[0] or dynamic[1] is not self.dynamic_scale[1]:
            keep: list = []
            descs = [ctypes.byref(_desc(t, keep)) if t is not None else None for t in dynamic]
            check_raf(_lib.dialect().rafhip_raf_env_set_dynamic_scale(self.handle, *descs))
            self.dynamic_scale = tuple(dynamic)

    def __del__(self):
        try:
            _lib.dialect().rafhip_raf_env_destroy(self.handle)
        except Exception:
            pass


def _workspace(env: "_Env", like: torch.Tensor, stream) -> runtime.Memory:
    """The OpEnv's workspace requests as one chunk from the device's memory pool, allocated on the
    call's stream like the VM does around Execute (src/impl/vm/vm.cc:1099-1105, :846-853).  The
    chunk is kept with the OpEnv and reused by later calls on the same stream (which run after this
    one): on ROCm 7.2 a stream-ordered allocation waits for the stream's pending work, which would
    serialise host and device once per step."""
    ws = env.workspaces.get(stream)
    if ws is None:
        dev_id = like.device.index if like.device.index is not None else 0
        ws = env.workspaces[stream] = runtime.Memory(DEV_ROCM, dev_id, env.workspace_bytes, 256, stream,
                                                     stream_ordered=True)
    return ws


class _EnvCache(collections.OrderedDict):
    """OpEnvs by call signature, the least recently used dropped beyond `capacity`: every OpEnv owns
    device tables, pinned staging memory and a workspace per stream, and hyper-parameters other than
    the learning rate are part of the signature, so an unbounded table would grow with every new
    value a training script tries."""

    capacity = 64

    def get(self, key, default=None):
        env = super().get(key, default)
        if env is not default:
            self.move_to_end(key)
        return env

    def __setitem__(self, key, env):
        super().__setitem__(key, env)
        self.move_to_end(key)
        while len(self) > self.capacity:
            self.popitem(last=False)


_env_cache = _EnvCache()


def clear_op_env_cache() -> None:
    _env_cache.clear()
    _recent_lists.clear()


class TensorList:
    """A tensor list held the way RAF's callers hold one: as an immutable tuple value
    (``TupleValue`` of ``TensorValue``s, include/raf/value.h).  The descriptors, the addresses and
    the C++ tuple are made once; ``lans`` / ``lans_mixed`` / ``sgd_multi`` accept the handle
    wherever they accept a list, and a call with it marshals nothing.

    The handle records where the tensors' storage was when it was made.  Unless ``track=False``
    every use checks, in one pass at C speed, that each tensor still lives there (``x.data = ...``,
    ``set_()`` and ``resize_()`` move a tensor without replacing the Python object) and rebuilds
    the handle if not, so it is never silently stale; ``rebuilds`` counts that.  With
    ``track=False`` the caller vouches for it, as for a ``TupleValue``, which nothing re-reads.
    Either way the handle keeps the tensors alive."""

    def __init__(self, tensors, track: bool = True, _share=None):
        self._tensors = list(tensors)
        self.track = bool(track)
        self.rebuilds = 0
        self.rebinds = 0
        self._volatile = None  # the (first, end) stretch whose tensors are new at every call, once known
        self._handle = c_void_p(None)
        self._build(_share)

    def _build(self, share=None) -> None:
        lib, glue = _lib.dialect(), _lib.glue()
        n = len(self._tensors)
        if share is None:
            self._descs = (TensorDesc * max(n, 1))()
            self._ptrs = (ctypes.c_uint64 * max(n, 1))()
            self._shapes = (c_int64 * max(8 * n, 1))()
            try:
                glue.describe(self._tensors, ctypes.addressof(self._descs), ctypes.addressof(self._shapes),
                              len(self._shapes), ctypes.addressof(self._ptrs))
            except ValueError as e:
                if "shape buffer" not in str(e):
                    raise
                self._shapes = (c_int64 * max(sum(t.dim() for t in self._tensors), 1))()
                glue.describe(self._tensors, ctypes.addressof(self._descs), ctypes.addressof(self._shapes),
                              len(self._shapes), ctypes.addressof(self._ptrs))
            h = c_void_p(None)
            check_raf(lib.rafhip_raf_tuple_make(n, self._descs, ctypes.byref(h)))
        else:
            # Everything outside [first, end) is the other handle's: its descriptors are copied, its
            # tensor values shared; only the fields in the range are described and made anew.
            base, first, end = share
            k = end - first
            self._descs = (TensorDesc * max(n, 1))()
            ctypes.memmove(self._descs, base._descs, ctypes.sizeof(TensorDesc) * n)
            self._ptrs = (ctypes.c_uint64 * max(n, 1))()
            ctypes.memmove(self._ptrs, base._ptrs, 8 * n)
            part = (c_int64 * max(8 * k, 1))()
            glue.describe(self._tensors[first:end], ctypes.addressof(self._descs) + ctypes.sizeof(TensorDesc) * first,
                          ctypes.addressof(part), len(part), ctypes.addressof(self._ptrs) + 8 * first)
            self._shapes = (base._shapes, part)  # both stay alive: the descriptors point into them
            h = c_void_p(None)
            check_raf(lib.rafhip_raf_tuple_replace(base._handle, first, k,
                                                   ctypes.cast(ctypes.addressof(self._descs) +
                                                               ctypes.sizeof(TensorDesc) * first,
                                                               ctypes.POINTER(TensorDesc)), ctypes.byref(h)))
        old, self._handle = self._handle, h
        if old:
            lib.rafhip_raf_tuple_destroy(old)
        # What identifies an OpEnv made for this list: every tensor's dtype, device and shape.  A
        # bytes object, so that a dictionary compares two lists' signatures with one memcmp and
        # the handle's own signature by identity.
        self.signature = glue.signature(ctypes.addressof(self._descs), n)

    def current(self) -> bool:
        """Whether every tensor's storage is where it was when the handle was made."""
        return _lib.glue().same_storage(self._tensors, ctypes.addressof(self._ptrs))

    def refresh(self) -> "TensorList":
        """Brings the handle up to date with its tensors if their storage moved."""
        if not self.current():
            self._build()
            self.rebuilds += 1
        return self

    def replaced(self, first: int, tensors) -> "TensorList":
        """A new handle that differs from this one in the tensors from ``first`` on (as many as
        given): the list of the next step when, say, only the gradients were allocated anew."""
        tensors = list(tensors)
        end = first + len(tensors)
        if first < 0 or end > len(self._tensors):
            raise IndexError("replacement range outside the list")
        merged = self._tensors[:first] + tensors + self._tensors[end:]
        return TensorList(merged, self.track, _share=(self, first, end))

    def _rebind(self, tensors: list, first: int, end: int) -> bool:
        """Takes over ``tensors``, which differ from this handle's in [first, end), in place: the
        tuple's tensor values of that range are rebound to the new storage, the way the
        reference's ``ndarray.update`` rebinds an array (python/raf/_core/ndarray.py:191-195).
        Only for a handle that no caller holds.  False, with nothing changed, if a tensor of the
        range differs in dtype, device or shape, a tensor outside it has moved, or something
        still shares the tuple."""
        if not _lib.glue().rebind(tensors, first, end, ctypes.addressof(self._descs), ctypes.addressof(self._ptrs)):
            return False
        done = ctypes.c_int32(0)
        fields = ctypes.cast(ctypes.addressof(self._descs) + ctypes.sizeof(TensorDesc) * first,
                             ctypes.POINTER(TensorDesc))
        check_raf(_lib.dialect().rafhip_raf_tuple_rebind(self._handle, first, end - first, fields,
                                                         ctypes.byref(done)))
        if not done.value:  # the descriptors already name the new storage: make the tuple anew from them
            h = c_void_p(None)
            check_raf(_lib.dialect().rafhip_raf_tuple_make(len(tensors), self._descs, ctypes.byref(h)))
            old, self._handle = self._handle, h
            _lib.dialect().rafhip_raf_tuple_destroy(old)
        self._tensors = list(tensors)
        self.rebinds += 1
        return True

    def _release_volatile(self) -> None:
        """After a call: lets go of the tensors in the stretch that is new at every call (the
        gradients of the step just enqueued).  Holding them until the next call would keep a whole
        generation of gradients allocated through the next forward and backward pass; the kernels
        already enqueued are ordered in front of any reuse of that memory by the stream."""
        if self._volatile is not None:
            first, end = self._volatile
            self._tensors[first:end] = [None] * (end - first)

    def __len__(self):
        return len(self._tensors)

    def __getitem__(self, i):
        return self._tensors[i]

    def __iter__(self):
        return iter(self._tensors)

    def __del__(self):
        try:
            if self._handle:
                _lib.dialect().rafhip_raf_tuple_destroy(self._handle)
        except Exception:
            pass


_recent_lists: "collections.deque[TensorList]" = collections.deque(maxlen=8)


def _tensor_list(tensors) -> TensorList:
    """The handle behind a ``tensor_list`` argument.  A ``TensorList`` is used as it is (checked
    against its tensors unless it was made with ``track=False``).  A plain sequence is looked up
    among the handles made for recent calls by the identity of its elements -- a training loop
    passes the same tensor objects every step.  When only a stretch of it differs from a recent
    list, what happens depends on whether the old tensors of that stretch can come back: if
    nothing but the handle refers to them any more (gradients that autograd allocates per
    iteration), the handle takes the new ones over in place and stops holding on to that stretch
    between calls; if the caller still has them (it alternates between lists), a new handle shares
    the rest with the old one, and once there are eight the oldest is taken over."""
    if isinstance(tensors, TensorList):
        return tensors.refresh() if tensors.track else tensors
    lst = tensors if type(tensors) is list else list(tensors)
    glue = _lib.glue()
    nearest = None
    for h in _recent_lists:
        if len(h) != len(lst):
            continue
        first, end = glue.diff_range(lst, h._tensors)
        if first < 0:
            if h is not _recent_lists[0]:
                _recent_lists.remove(h)
                _recent_lists.appendleft(h)
            return h.refresh()
        if 2 * (end - first) <= len(lst) and (nearest is None or end - first < nearest[2] - nearest[1]):
            nearest = (h, first, end)

    def take_over(h, first, end):
        if not h._rebind(lst, first, end):
            return False
        if h is not _recent_lists[0]:
            _recent_lists.remove(h)
            _recent_lists.appendleft(h)
        return True

    if nearest is not None:
        h, first, end = nearest
        # Tensors that are new at every call (gradients allocated per iteration, torch's default):
        # when nothing but the handle still refers to the ones it holds in the stretch, nobody can
        # pass them again, so the handle takes the new ones over in place -- and from then on lets
        # go of that stretch after every call instead of keeping a generation of gradients alive.
        if h._volatile is not None or glue.unreferenced(h._tensors, first, end):
            if take_over(h, first, end):
                lo, hi = h._volatile or (first, end)
                h._volatile = (min(lo, first), max(hi, end))
                return h
        elif len(_recent_lists) == _recent_lists.maxlen:
            # The caller keeps the old tensors (it may alternate between a few lists, which are all
            # found above) but brings new ones again and again: rather than make handle after
            # handle, the one used longest ago takes the new tensors over.
            for old in reversed(_recent_lists):
                if len(old) != len(lst) or old._volatile is not None:
                    continue
                first2, end2 = glue.diff_range(lst, old._tensors)
                if 2 * (end2 - first2) <= len(lst) and take_over(old, first2, end2):
                    return old
                break
    if nearest is not None and nearest[0]._volatile is None and nearest[0].current():
        h = nearest[0].replaced(nearest[1], lst[nearest[1]:nearest[2]])
    else:
        h = TensorList(lst)
    _recent_lists.appendleft(h)
    return h


def _sig(t: torch.Tensor):
    return (tuple(t.shape), t.dtype, str(t.device))


def sgd(x, dx, v, learning_rate, mu):
    """``raf._op.imp.sgd(x, dx, v, learning_rate, mu) -> (v1, x1)``: new tensors, inputs untouched
    (src/op/declare/optimizer.cc:22-44)."""
    lib = _lib.dialect()
    keep: list = []
    dx_, ddx, dv = _desc(x, keep), _desc(dx, keep), _desc(v, keep)
    key = ("sgd", _sig(x), _sig(dx), _sig(v), float(mu))
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        check_raf(lib.rafhip_raf_sgd_make(dx_, ddx, dv, float(learning_rate), float(mu),
                                          ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
        env.learning_rate = float(learning_rate)
    env.set_learning_rate(float(learning_rate))
    v1 = torch.empty_like(dx)  # the executor's AllocOutputBuffer (interpreter.cc:397-426)
    x1 = torch.empty_like(dx)
    check_raf(lib.rafhip_raf_sgd_execute(env.handle, dx_, ddx, dv, _desc(v1, keep), _desc(x1, keep),
                                         _stream(dx)))
    return v1, x1


class TracedSgdUpdate:
    """The per-parameter update of the reference's traced SGD optimizer,
    ``add(multiply(momentum, v), dx, out=v)`` then ``subtract(w, multiply(learning_rate, new_v),
    out=w)`` with ``cast(dx, "float32")`` in front for a 16-bit gradient
    (python/raf/optim/sgd.py:192-200), taken through the dialect fusion pass: the graph is built,
    the ``hip`` dialect's ``sgd_update`` pattern turns it into one primitive function, and every
    call of this object runs that function as one kernel launch, in place on ``w`` and ``v``.
    The tensors are bound once, as a traced model binds its parameters; ``ir_before`` / ``ir_after``
    hold the text of the graph on either side of the pass."""

    def __init__(self, w, dx, v, learning_rate, momentum):
        lib = _lib.dialect()
        self._keep: list = [w, dx, v]
        self._descs = (_desc(w, self._keep), _desc(dx, self._keep), _desc(v, self._keep))
        self.w = w
        key = ("traced_sgd", _sig(w), _sig(dx), _sig(v), float(learning_rate), float(momentum))
        env = _env_cache.get(key)
        if env is None:
            h = c_void_p(None)
            status = lib.rafhip_raf_traced_sgd_make(*self._descs, float(learning_rate), float(momentum),
                                                    ctypes.byref(h))
            made = _Env(h) if h.value else None  # also set when nothing fused: it then holds the graphs
            check_raf(status)
            env = _env_cache[key] = made
        self._env = env
        self._execute = lib.rafhip_raf_traced_sgd_execute

    def __call__(self):
        check_raf(self._execute(self._env.handle, *self._descs, _stream(self.w)))
        return self.w

    def _text(self, fused: int) -> str:
        buf = ctypes.create_string_buffer(1 << 14)
        check_raf(_lib.dialect().rafhip_raf_env_ir_text(self._env.handle, fused, buf, len(buf)))
        return buf.value.decode()

    @property
    def ir_before(self) -> str:
        return self._text(0)

    @property
    def ir_after(self) -> str:
        return self._text(1)

    @property
    def op(self) -> str:
        return self._env.op


def traced_sgd_update(w, dx, v, learning_rate, momentum, return_ir=False):
    """One fused traced update (see ``TracedSgdUpdate``) of ``w`` and ``v`` in place; returns ``w``
    (the traced ``new_w`` shares its memory), with ``return_ir`` also the graph text before and
    after the pass."""
    upd = TracedSgdUpdate(w, dx, v, learning_rate, momentum)
    upd()
    return (w, upd.ir_before, upd.ir_after) if return_ir else w


class _TracedOptimizer:
    """Common part of the two traced optimizers below: the optimizer graph is built for the given
    parameter lists, taken through the FuseDialect pass (the hip dialect's graph rewrites first,
    its patterns after), and every call of the resulting graph gets an OpEnv; ``__call__`` runs them
    in order, in place on the tensors.  ``ir_before`` / ``ir_after`` hold the graph's text on either
    side of the pass, ``ops`` what the fused graph calls (a leading ``!`` marks an operator that
    stayed unfused and has no backend here)."""

    _KIND = None

    def _make(self, lists, step, zero_is_constant, hyper, allow_partial):
        lib = _lib.dialect()
        self._keep: list = [lists, step]
        self._n = len(lists[1])
        self._allow_partial = int(bool(allow_partial))

        def array(ts):
            if ts is None:
                return None
            if len(ts) != self._n:
                raise ValueError("the tensor lists differ in length")
            return (TensorDesc * max(self._n, 1))(*[_desc(t, self._keep) for t in ts])

        self._descs = [array(ts) for ts in lists]
        self._step = ctypes.byref(_desc(step, self._keep)) if step is not None else None
        hy = (ctypes.c_double * len(hyper))(*[float(x) for x in hyper])
        h = c_void_p(None)
        status = lib.rafhip_raf_traced_optimizer_make(self._KIND, self._n, *self._descs, self._step,
                                                      int(bool(zero_is_constant)), hy, len(hyper),
                                                      self._allow_partial, ctypes.byref(h))
        self._env = _Env(h) if h.value else None  # also set on failure: it then holds the graphs
        check_raf(status)
        self._first = lists[1][0]
        self._execute = lib.rafhip_raf_traced_optimizer_execute

    def __call__(self):
        stream = _stream(self._first)
        if self._KIND == 1:  # the loss scaling in force reaches the LANS call of the graph
            self._env.set_grad_scaling(_lans_grad_unscale, _lans_dynamic_scale)
        ws = _workspace(self._env, self._first, stream) if self._env.workspace_bytes > 0 else None
        check_raf(self._execute(self._env.handle, self._n, *self._descs, self._step, self._allow_partial,
                                ws.data if ws else None, self._env.workspace_bytes, stream))

    def _text(self, fused: int) -> str:
        buf = ctypes.create_string_buffer(1 << 22)
        check_raf(_lib.dialect().rafhip_raf_env_ir_text(self._env.handle, fused, buf, len(buf)))
        return buf.value.decode()

    @property
    def ir_before(self) -> str:
        return self._text(0)

    @property
    def ir_after(self) -> str:
        return self._text(1)

    @property
    def ops(self) -> List[str]:
        buf = ctypes.create_string_buffer(1 << 16)
        check_raf(_lib.dialect().rafhip_raf_env_graph_ops(self._env.handle, buf, len(buf)))
        return [x for x in buf.value.decode().split(";") if x]


class TracedSgdOptimizer(_TracedOptimizer):
    """The optimizer part of what the reference's traced SGD optimizer builds for a whole model
    (python/raf/optim/sgd.py:187-215): per parameter ``add(multiply(momentum, v), dx, out=v)`` and
    ``subtract(w, multiply(learning_rate, new_v), out=w)`` (with ``cast(dx, "float32")`` in front
    for a 16-bit gradient) and, with ``p`` (a half-precision model with fp32 master weights ``w``),
    ``add(cast(new_w, dtype), zero, out=p)``.  The hip dialect gathers all of it into one
    multi-tensor call.  ``zero_is_constant=False`` leaves the optimizer's zero tensor a free
    variable, as traced: the cast and the copy then stay unfused (and, with ``allow_partial``, are
    left out when the graph is run, since this library has no backend for them)."""

    _KIND = 0

    def __init__(self, w, dx, v, learning_rate, momentum, p=None, zero_is_constant=True, allow_partial=False):
        self._make([list(dx), list(w), None, list(v), list(p) if p is not None else None], None,
                   zero_is_constant, [learning_rate, momentum], allow_partial)


class TracedLansOptimizer(_TracedOptimizer):
    """The optimizer part of what the reference's traced LANS optimizer builds for a half-precision
    model (python/raf/optim/lans.py:244-312): ``group_cast(g, "float32")``, ``raf.op.lans`` over
    ``[g32..., w..., m..., v...]``, and per parameter ``cast(new_w, dtype)`` and
    ``add(_, zero, out=p)``.  The hip dialect folds all of it into one ``raf.op.hip.lans_mixed``
    call; with ``zero_is_constant=False`` only the group_cast folds (``raf.op.hip.lans`` on the half
    gradients)."""

    _KIND = 1

    def __init__(self, g, w, m, v, p, step, learning_rate=1e-3, beta1=0.9, beta2=0.999, eps=1e-6,
                 bias_correction=True, weight_decay=0.01, grad_averaging=True, mode=True, normalize_grad=True,
                 zero_is_constant=True, allow_partial=False):
        self._make([list(g), list(w), list(m), list(v), list(p)], step, zero_is_constant,
                   [learning_rate, beta1, beta2, eps, int(bias_correction), weight_decay, int(grad_averaging),
                    int(mode), int(bool(normalize_grad))], allow_partial)


def sgd_multi(tensor_list: Sequence[torch.Tensor], learning_rate, mu):
    """Extension op: momentum SGD over a parameter list ``[x..., dx..., v...]`` in place (x and v
    are updated, the list is returned), one launch; per element the four roundings of ``sgd``."""
    return _sgd_multi(False, tensor_list, learning_rate, mu)


def sgd_multi_mixed(tensor_list: Sequence[torch.Tensor], learning_rate, mu):
    """Extension op for half-precision models: ``[x..., dx..., v..., p...]`` with fp32 master weights
    ``x``, gradients of the model's dtype and the model's float16 / bfloat16 parameters ``p``, which
    receive the new weights narrowed to 16 bits (python/raf/optim/sgd.py:187-215 in one op)."""
    return _sgd_multi(True, tensor_list, learning_rate, mu)


def _sgd_multi(mixed, tensor_list, learning_rate, mu):
    lib = _lib.dialect()
    tl = _tensor_list(tensor_list)
    n = len(tl)
    key = ("sgd_multi", mixed, tl.signature, float(mu))
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        check_raf(lib.rafhip_raf_sgd_multi_make(int(mixed), n, tl._descs, float(learning_rate), float(mu),
                                                ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
        env.learning_rate = float(learning_rate)
    if n:
        env.set_learning_rate(float(learning_rate))
    check_raf(lib.rafhip_raf_sgd_multi_execute_tuple(env.handle, tl._handle, _stream(tl[0]) if n else None, _as_vm))
    tl._release_volatile()
    return tensor_list


def lans(tensor_list: Sequence[torch.Tensor], step: torch.Tensor, learning_rate, beta1, beta2, eps,
         bias_correction, weight_decay, grad_averaging, mode, normalize_grad):
    """``raf._op.imp.lans(...)``: updates the w, m, v quarters of ``tensor_list`` in place and
    returns the list (the op's output aliases its input, declare/optimizer.cc:53-57).  Booleans
    become ints as the schema's ``int`` fields receive them (python/raf/optim/lans.py:51-54)."""
    return _lans("lans", tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction,
                 weight_decay, grad_averaging, mode, normalize_grad)


def lans_mixed(tensor_list: Sequence[torch.Tensor], step: torch.Tensor, learning_rate, beta1, beta2,
               eps, bias_correction, weight_decay, grad_averaging, mode, normalize_grad):
    """Extension op for half-precision models with fp32 master weights: ``tensor_list`` holds five
    blocks ``[g..., w..., m..., v..., p...]``; ``p`` are the model's float16 / bfloat16 parameters
    and receive the new weights narrowed to 16 bits.  One call does what the reference's traced
    optimizer builds from ``group_cast`` + ``lans`` + ``cast`` + ``add(out=p)``
    (python/raf/optim/lans.py:261-265, :289-291, :303-305)."""
    return _lans("lans_mixed", tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction,
                 weight_decay, grad_averaging, mode, normalize_grad)


def _lans(op_name, tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction,
          weight_decay, grad_averaging, mode, normalize_grad):
    lib = _lib.dialect()
    keep: list = []
    tl = _tensor_list(tensor_list)
    n4 = len(tl)
    dstep = _desc(step, keep)
    hp = (float(learning_rate), float(beta1), float(beta2), float(eps), int(bias_correction),
          float(weight_decay), int(grad_averaging), int(mode), int(bool(normalize_grad)))
    # All but the learning rate and the loss scaling.  Lists of equal signature (two models of one
    # architecture) share an OpEnv: its plan keeps a device pointer table per recent list.
    key = (op_name, tl.signature, _sig(step), hp[1:])
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        make = lib.rafhip_raf_lans_make if op_name == "lans" else lib.rafhip_raf_lans_mixed_make
        check_raf(make(n4, tl._descs, dstep, *hp, ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
        env.learning_rate = hp[0]
    if n4:
        env.set_learning_rate(hp[0])
        env.set_grad_scaling(_lans_grad_unscale, _lans_dynamic_scale)
    stream = _stream(tl[0]) if n4 else None
    ws = _workspace(env, tl[0], stream) if env.workspace_bytes > 0 else None
    check_raf(lib.rafhip_raf_lans_execute_tuple(env.handle, tl._handle, dstep, ws.data if ws else None,
                                                env.workspace_bytes, stream, _as_vm))
    tl._release_volatile()
    return tensor_list


_TORCH_DTYPES = {v: k for k, v in _DTYPES.items()}


def _alloc_outputs(env: _Env, device) -> List[torch.Tensor]:
    """Allocate what the op's declare function produced, like the executor's AllocOutputBuffer
    (src/impl/interpreter.cc:397-426)."""
    lib = _lib.dialect()
    outs = []
    for i in range(lib.rafhip_raf_env_num_outputs(env.handle)):
        code, bits, ndim = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
        shape = (c_int64 * 16)()
        check_raf(lib.rafhip_raf_env_output(env.handle, i, ctypes.byref(code), ctypes.byref(bits),
                                            ctypes.byref(ndim), shape, 16))
        outs.append(torch.empty(tuple(shape[:ndim.value]), dtype=_TORCH_DTYPES[(code.value, bits.value)],
                                device=device))
    return outs


def l2norm(x: torch.Tensor) -> torch.Tensor:
    """``raf._op.imp.l2norm(x)``: sqrt(sum(x*x)) as a 0-d tensor of x's dtype on x's device
    (src/op/declare/reduce.cc:118-124)."""
    lib = _lib.dialect()
    keep: list = []
    dx = _desc(x, keep)
    key = ("l2norm", _sig(x))
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        check_raf(lib.rafhip_raf_l2norm_make(dx, ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
    (out,) = _alloc_outputs(env, x.device)
    ws = _workspace(env, x, _stream(x)) if env.workspace_bytes else None
    check_raf(lib.rafhip_raf_l2norm_execute(env.handle, dx, _desc(out, keep), ws.data if ws else None,
                                            env.workspace_bytes, _stream(x)))
    return out


def fuse_tensor(data: Sequence[torch.Tensor]):
    """``raf._op.imp.fuse_tensor(data)``: one flat 1-d tensor with every tensor's elements back to
    back (src/op/declare/memory.cc:43-63).  An empty list has no output (None)."""
    lib = _lib.dialect()
    data = list(data)
    keep: list = []
    descs = (TensorDesc * max(len(data), 1))(*[_desc(t, keep) for t in data])
    key = ("fuse_tensor", tuple(_sig(t) for t in data))
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        check_raf(lib.rafhip_raf_fuse_tensor_make(len(data), descs, ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
    if not data:
        return None
    (out,) = _alloc_outputs(env, data[0].device)
    check_raf(lib.rafhip_raf_fuse_tensor_execute(env.handle, len(data), descs, _desc(out, keep), _stream(data[0])))
    return out


def defuse_tensor(data: torch.Tensor, sizes, shapes, shape_indices):
    """``raf._op.imp.defuse_tensor(data, sizes, shapes, shape_indices)``: the inverse of
    ``fuse_tensor``; ``sizes`` are element counts, ``shapes`` the concatenated dimensions and
    ``shape_indices`` where each output's dimensions end (src/op/declare/memory.cc:65-93)."""
    lib = _lib.dialect()
    keep: list = []
    dd = _desc(data, keep)
    sizes, shapes, shape_indices = [int(v) for v in sizes], [int(v) for v in shapes], [int(v) for v in shape_indices]
    key = ("defuse_tensor", _sig(data), tuple(sizes), tuple(shapes), tuple(shape_indices))
    env = _env_cache.get(key)
    if env is None:
        h = c_void_p(None)
        arr = lambda v: (c_int64 * max(len(v), 1))(*v)
        check_raf(lib.rafhip_raf_defuse_tensor_make(dd, len(sizes), arr(sizes), len(shapes), arr(shapes),
                                                    len(shape_indices), arr(shape_indices), ctypes.byref(h)))
        env = _env_cache[key] = _Env(h)
    outs = _alloc_outputs(env, data.device)
    descs = (TensorDesc * max(len(outs), 1))(*[_desc(t, keep) for t in outs])
    check_raf(lib.rafhip_raf_defuse_tensor_execute(env.handle, dd, len(outs), descs, _stream(data)))
    return outs


_lans_grad_unscale = 1.0
_lans_dynamic_scale = (None, None)
_as_vm = 0


def set_executor(kind: str) -> None:
    """Which of RAF's executors the multi-tensor ops imitate when they hand a tensor list to an
    OpEnv: "interpreter" passes the list's tuple value itself (src/impl/interpreter.cc:286-325),
    "vm" a newly allocated ``TupleValue`` over the same tensor values at every call, which is what
    the VM's AllocTuple instruction produces per iteration (src/impl/vm/vm.cc:764-769)."""
    global _as_vm
    _as_vm = {"interpreter": 0, "vm": 1}[kind]


def set_lans_grad_unscale(factor: float) -> None:
    """hip-dialect extension: LANS multiplies every gradient by ``factor`` first (e.g. 1/1024 to
    undo a loss scale on fp16 gradients).  Applies to every LANS call from now on; OpEnvs are kept."""
    global _lans_grad_unscale
    _lans_grad_unscale = float(factor)


def get_lans_grad_unscale() -> float:
    return _lans_grad_unscale


def set_lans_dynamic_scale(grad_unscale: torch.Tensor = None, found_inf: torch.Tensor = None) -> None:
    """hip-dialect extension for dynamic loss scaling: 0-d float32 GPU tensors holding the
    reciprocal of the current loss scale (it replaces the static factor) and the overflow flag (a
    non-zero value makes the LANS step a no-op).  The kernels read both on the device, so the scale
    can change and a step can be skipped without a host synchronisation or a new OpEnv.  ``None``
    switches either off."""
    global _lans_dynamic_scale
    for t, name in ((grad_unscale, "grad_unscale"), (found_inf, "found_inf")):
        if t is not None and (not isinstance(t, torch.Tensor) or t.dtype != torch.float32 or t.numel() != 1
                              or not t.is_cuda):
            raise TypeError(f"{name} must be a one-element float32 GPU tensor")
    _lans_dynamic_scale = (grad_unscale, found_inf)


def serve_stream_requests(enable: bool) -> None:
    """Whether this thread's executor stand-in serves ``OpEnv::RequestStream`` (include/raf/op.h:87):
    with it, ``fuse_tensor`` / ``defuse_tensor`` run on the copy stream they request, as the
    reference's do (src/op/dialect/cuda/memory.cc:34, :89), ordered behind the current stream
    before and in front of it after; without it (the default) they run on the current stream."""
    check_raf(_lib.dialect().rafhip_raf_serve_stream_requests(int(bool(enable))))


def get_lans_dynamic_scale():
    """The (grad_unscale, found_inf) tensors in force, either of them possibly None."""
    return _lans_dynamic_scale


def dispatch_list(base_op: str, device_type: int = DEV_ROCM) -> List[Tuple[str, str, int]]:
    """[(dialect, dialect_op, plevel)] in dispatch order (OpDialect::GetDispatchList)."""
    buf = ctypes.create_string_buffer(4096)
    check_raf(_lib.dialect().rafhip_raf_dispatch_list(base_op.encode(), device_type, buf, 4096))
    out = []
    for item in buf.value.decode().split(";"):
        if item:
            d, o, p = item.split(":")
            out.append((d, o, int(p)))
    return out


class with_dialect:
    """Context manager pinning the dialects dispatch may use, like the reference's test helper
    ``raf.testing.with_dialect`` (python/raf/testing/common.py:260-278)."""

    def __init__(self, dialects):
        self.dialects = [dialects] if isinstance(dialects, str) else list(dialects)

    def __enter__(self):
        check_raf(_lib.dialect().rafhip_raf_set_dialect_preference(",".join(self.dialects).encode()))
        return self

    def __exit__(self, *exc):
        check_raf(_lib.dialect().rafhip_raf_set_dialect_preference(None))
        return False
