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
