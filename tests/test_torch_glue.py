"""The CPython module that reads lists of torch tensors for the operator front end, on the CPU:
what it writes must be what the per-tensor Python marshalling (`raf_amd.op._desc`) writes."""
import ctypes

import pytest
import torch


def _describe(glue, tensors):
    from raf_amd._lib import TensorDesc

    n = len(tensors)
    descs = (TensorDesc * max(n, 1))()
    ptrs = (ctypes.c_uint64 * max(n, 1))()
    shapes = (ctypes.c_int64 * max(8 * n, 1))()
    used = glue.describe(tensors, ctypes.addressof(descs), ctypes.addressof(shapes), len(shapes),
                         ctypes.addressof(ptrs))
    return descs, ptrs, shapes, used


def test_describe_agrees_with_the_python_marshalling(native_libs):
    from raf_amd import op

    glue = native_libs.glue()
    tensors = [torch.zeros(3, 5), torch.zeros((), dtype=torch.float16), torch.zeros(7, dtype=torch.bfloat16),
               torch.zeros(2, 2, 2, dtype=torch.float64), torch.zeros(0), torch.zeros(4, dtype=torch.int32),
               torch.zeros(9, dtype=torch.int64), torch.zeros(1, dtype=torch.uint8), torch.arange(12.0)[4:]]
    descs, ptrs, _, used = _describe(glue, tensors)
    assert used == sum(t.dim() for t in tensors)
    for i, t in enumerate(tensors):
        keep = []
        want = op._desc(t, keep)
        got = descs[i]
        assert (got.data or 0) == (want.data or 0) == t.data_ptr() == ptrs[i]
        assert (got.device_type, got.device_id, got.dtype_code, got.dtype_bits, got.ndim) == (
            want.device_type, want.device_id, want.dtype_code, want.dtype_bits, want.ndim)
        assert list(got.shape[:got.ndim]) == list(t.shape)


def test_describe_refuses_what_the_operators_cannot_take(native_libs):
    glue = native_libs.glue()
    with pytest.raises(ValueError, match="contiguous"):
        _describe(glue, [torch.zeros(4, 4).t()])
    with pytest.raises(TypeError, match="expected a tensor"):
        _describe(glue, [torch.zeros(1), 3.0])
    with pytest.raises(TypeError, match="dtype"):
        _describe(glue, [torch.zeros(2, dtype=torch.complex64)])
    with pytest.raises(TypeError, match="must be a list"):
        glue.same_storage((torch.zeros(1),), 0)


def test_same_storage_sees_every_way_a_tensor_can_move(native_libs):
    glue = native_libs.glue()
    tensors = [torch.zeros(16) for _ in range(50)]
    _, ptrs, _, _ = _describe(glue, tensors)
    addr = ctypes.addressof(ptrs)
    assert glue.same_storage(tensors, addr)
    tensors[49].data = torch.zeros(16)
    assert not glue.same_storage(tensors, addr)
    _, ptrs, _, _ = _describe(glue, tensors)
    addr = ctypes.addressof(ptrs)
    tensors[0].set_(torch.zeros(16))
    assert not glue.same_storage(tensors, addr)
    _, ptrs, _, _ = _describe(glue, tensors)
    addr = ctypes.addressof(ptrs)
    tensors[7].resize_(1 << 16)  # beyond the storage: reallocated
    assert not glue.same_storage(tensors, addr)
    # writes in place do not move anything
    _, ptrs, _, _ = _describe(glue, tensors)
    tensors[3].add_(1.0)
    assert glue.same_storage(tensors, ctypes.addressof(ptrs))


def test_diff_range_and_signature(native_libs):
    from raf_amd._lib import TensorDesc

    glue = native_libs.glue()
    a = [torch.zeros(2) for _ in range(10)]
    assert glue.diff_range(a, list(a)) == (-1, -1)
    b = list(a)
    b[3] = torch.zeros(2)
    assert glue.diff_range(a, b) == (3, 4)
    b[6] = torch.zeros(2)
    assert glue.diff_range(a, b) == (3, 7)
    with pytest.raises(ValueError):
        glue.diff_range(a, a[:5])
    d1, _, s1, _ = _describe(glue, [torch.zeros(2, 3), torch.zeros(4)])
    d2, _, s2, _ = _describe(glue, [torch.ones(2, 3), torch.ones(4)])
    d3, _, s3, _ = _describe(glue, [torch.zeros(3, 2), torch.zeros(4)])
    d4, _, s4, _ = _describe(glue, [torch.zeros(2, 3), torch.zeros(4, dtype=torch.float16)])
    sig = lambda d: glue.signature(ctypes.addressof(d), 2)
    assert sig(d1) == sig(d2)            # values and addresses are no part of it
    assert sig(d1) != sig(d3) and sig(d1) != sig(d4)
    assert ctypes.sizeof(TensorDesc) == 40  # the layout torch_glue.cpp writes (rafhip_dialect.h)


def test_tensor_list_handle_on_the_cpu(native_libs):
    """The handle itself needs no GPU: making, tracking, replacing."""
    from raf_amd import op

    ts = [torch.zeros(3, 5) for _ in range(12)]
    tl = op.TensorList(ts)
    assert len(tl) == 12 and tl[4] is ts[4] and list(tl) == ts and tl.current()
    ts[5].data = torch.ones(3, 5)
    assert not tl.current()
    assert tl.refresh() is tl and tl.current() and tl.rebuilds == 1
    new = [torch.zeros(3, 5) for _ in range(3)]
    t2 = tl.replaced(0, new)
    assert t2 is not tl and t2[0] is new[0] and t2[3] is ts[3] and t2.signature == tl.signature
    assert native_libs.dialect().rafhip_raf_tuple_size(t2._handle) == 12
    with pytest.raises(IndexError):
        tl.replaced(11, new)
    with pytest.raises(TypeError):
        tl[0] = ts[1]
    # a plain list of the same objects finds the handle made for it; new objects in a stretch share the rest
    op.clear_op_env_cache()
    h = op._tensor_list(ts)
    assert op._tensor_list(list(ts)) is h
    h2 = op._tensor_list(new + ts[3:])
    assert h2 is not h and h2[5] is ts[5]
    assert op._tensor_list(ts) is h
    op.clear_op_env_cache()


def test_rebind_writes_only_what_fits(native_libs):
    """`rebind` brings a described list up to date with other tensors in a range: the addresses
    of the range are written if dtype, device and shape agree and the rest has not moved; nothing
    at all is written otherwise."""
    glue = native_libs.glue()
    ts = [torch.zeros(2, 3), torch.zeros(7), torch.zeros(4, dtype=torch.float16), torch.zeros(())]
    descs, ptrs, _shapes, _ = _describe(glue, ts)
    addr = lambda: (ctypes.addressof(descs), ctypes.addressof(ptrs))
    new = [torch.ones(2, 3), torch.ones(7)]
    assert glue.rebind(new + ts[2:], 0, 2, *addr()) is True
    assert [ptrs[i] for i in range(4)] == [t.data_ptr() for t in new + ts[2:]]
    assert descs[0].data == new[0].data_ptr() and descs[1].data == new[1].data_ptr()
    assert descs[2].data == ts[2].data_ptr() and descs[0].ndim == 2 and descs[0].shape[1] == 3
    before = [ptrs[i] for i in range(4)]
    for bad in ([torch.ones(3, 2), torch.ones(7)],                       # another shape
                [torch.ones(2, 3), torch.ones(7, dtype=torch.float64)],  # another dtype
                [torch.ones(2, 3), torch.ones(7, 1)],                    # another rank
                [torch.ones(3, 2).t(), torch.ones(7)]):                  # not contiguous
        assert glue.rebind(bad + ts[2:], 0, 2, *addr()) is False
        assert [ptrs[i] for i in range(4)] == before and descs[0].data == before[0]
    # a tensor outside the range that has moved since: refused as a whole
    moved = ts[3]
    moved.data = torch.ones(())
    assert glue.rebind([torch.ones(2, 3), torch.ones(7)] + ts[2:], 0, 2, *addr()) is False
    assert [ptrs[i] for i in range(4)] == before
    with pytest.raises(IndexError):
        glue.rebind(new + ts[2:], 3, 5, *addr())
    with pytest.raises(TypeError):
        glue.rebind(new + [None, None], 0, 2, *addr())


def test_lists_with_new_tensors_every_call_reuse_the_oldest_handle(native_libs):
    """Gradients allocated anew at every step: once the front end's few recent handles are all
    taken, the one used longest ago takes the new tensors over in place instead of a handle being
    made per step; lists that come back are still found, and a list that does not fit (another
    shape in the range) gets a handle of its own."""
    from raf_amd import op

    op.clear_op_env_cache()
    state = [torch.zeros(3, 5) for _ in range(9)]
    keep, handles = [], []
    cap = op._recent_lists.maxlen
    for step in range(cap + 4):
        g = [torch.zeros(3, 5) for _ in range(3)]
        keep.append(g)
        h = op._tensor_list(g + state)
        assert h[0] is g[0] and h[3] is state[0] and h._ptrs[2] == g[2].data_ptr() and h.current()
        assert native_libs.dialect().rafhip_raf_tuple_size(h._handle) == 12
        handles.append(h)
    assert len(set(map(id, handles[:cap]))) == cap            # a handle each while there is room
    assert all(any(h is e for e in handles[:cap]) for h in handles[cap:])  # then reuse
    assert handles[cap] is handles[0] and handles[cap].rebinds == 1
    assert len(op._recent_lists) == cap
    # the most recent lists are still found as they are
    assert op._tensor_list(keep[-1] + state) is handles[-1]
    assert op._tensor_list(keep[-2] + state) is handles[-2]
    # a range that does not fit the old descriptors: a handle made from scratch, nothing rebound
    rebinds = sum(h.rebinds for h in op._recent_lists)
    odd = op._tensor_list([torch.zeros(5, 3) for _ in range(3)] + state)
    assert odd.rebinds == 0 and sum(h.rebinds for h in op._recent_lists if h is not odd) <= rebinds
    assert odd[0].shape == (5, 3) and odd.signature != handles[-1].signature
    op.clear_op_env_cache()


def test_tuple_rebind_refuses_a_shared_tuple(native_libs):
    """The C window rebinds in place only what nothing else shares: a tuple whose fields another
    tuple shares (made from it by _replace) is left as it is."""
    from raf_amd import op
    from raf_amd._lib import TensorDesc, check_raf

    lib = native_libs.dialect()
    ts = [torch.zeros(4) for _ in range(6)]
    a = op.TensorList(ts)
    b = a.replaced(0, [torch.zeros(4), torch.zeros(4)])   # shares fields 2..5 with a
    keep: list = []
    fresh = [torch.ones(4), torch.ones(4)]
    descs = (TensorDesc * 2)(*[op._desc(t, keep) for t in fresh])
    done = ctypes.c_int32(-1)
    check_raf(lib.rafhip_raf_tuple_rebind(a._handle, 4, 2, descs, ctypes.byref(done)))
    assert done.value == 0                                 # fields 4, 5 are b's too
    check_raf(lib.rafhip_raf_tuple_rebind(a._handle, 0, 2, descs, ctypes.byref(done)))
    assert done.value == 1                                 # fields 0, 1 are a's alone
    wrong = (TensorDesc * 2)(*[op._desc(t, keep) for t in (torch.ones(4, 1), torch.ones(4))])
    check_raf(lib.rafhip_raf_tuple_rebind(a._handle, 0, 2, wrong, ctypes.byref(done)))
    assert done.value == 0
    assert lib.rafhip_raf_tuple_rebind(a._handle, 5, 2, descs, ctypes.byref(done)) != 0  # out of range
    del b


def test_grads_reads_every_parameters_gradient(native_libs):
    glue = native_libs.glue()
    ps = [torch.nn.Parameter(torch.zeros(3)) for _ in range(4)]
    assert glue.grads(ps) == ([None] * 4, 4)
    ps[1].grad = torch.ones(3)
    ps[3].grad = torch.full((3,), 2.0)
    got, missing = glue.grads(ps)
    assert missing == 2 and got[0] is None and got[2] is None
    assert got[1] is ps[1].grad and got[3] is ps[3].grad
    assert glue.grads([]) == ([], 0)
    with pytest.raises(AttributeError):
        glue.grads([object()])
    with pytest.raises(TypeError):
        glue.grads(tuple(ps))


def test_a_stretch_that_is_new_at_every_call_is_not_kept_alive(native_libs):
    """Gradients that nobody holds after a step (autograd allocates new ones per iteration): one
    handle serves every step, takes the new tensors over in place, and lets go of that stretch
    after each call, so no generation of gradients outlives its step because of the front end."""
    import gc
    import weakref

    from raf_amd import op

    glue = native_libs.glue()
    a = [torch.zeros(3), torch.zeros(3)]
    assert glue.unreferenced([torch.zeros(3), a[0]], 0, 1) is True    # only the list holds item 0
    assert glue.unreferenced([torch.zeros(3), a[0]], 0, 2) is False   # `a` holds item 1 as well
    with pytest.raises(IndexError):
        glue.unreferenced(a, 1, 3)

    op.clear_op_env_cache()
    state = [torch.zeros(3, 5) for _ in range(9)]
    first = op._tensor_list([torch.zeros(3, 5) for _ in range(3)] + state)
    first._release_volatile()                      # nothing is known to be volatile yet: a no-op
    assert first[0] is not None and first._volatile is None
    seen = []
    for step in range(5):
        g = [torch.full((3, 5), float(step)) for _ in range(3)]
        seen.append(weakref.ref(g[0]))
        h = op._tensor_list(g + state)
        assert h is first and h._volatile == (0, 3) and h.rebinds == step + 1
        assert h[0] is g[0] and h._ptrs[1] == g[1].data_ptr() and h._descs[2].data == g[2].data_ptr()
        h._release_volatile()                      # what op.lans / op.sgd_multi do after Execute
        assert h[0] is None and h[3] is state[0]
        del g
        gc.collect()
        assert seen[-1]() is None                  # the step's gradients are gone with the step
    assert len(op._recent_lists) == 1
    # the persistent tensors are still tracked: a moved one makes the next call build a new handle
    state[4].data = torch.ones(3, 5)
    h2 = op._tensor_list([torch.zeros(3, 5) for _ in range(3)] + state)
    assert h2 is not first and h2.current() and h2._ptrs[3 + 4] == state[4].data_ptr()
    op.clear_op_env_cache()
