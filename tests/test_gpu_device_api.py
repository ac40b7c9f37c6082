"""The rocm DeviceAPI and the memory pools on a real device, through the host layer's C API:
allocation, the three copy directions, streams and events, stream-ordered allocation from the HIP
memory pool, the page-unit pool's reuse of idle chunks, and an operator running on a pool
workspace."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _host_desc(a, keep):
    from raf_amd._lib import TensorDesc

    shape = (ctypes.c_int64 * 1)(a.size)
    keep.append(shape)
    return TensorDesc(a.ctypes.data, 1, 0, 1, 8, 1, ctypes.cast(shape, ctypes.POINTER(ctypes.c_int64)))


def _dev_desc(ptr, nbytes, keep):
    from raf_amd._lib import TensorDesc

    shape = (ctypes.c_int64 * 1)(nbytes)
    keep.append(shape)
    return TensorDesc(ptr, 10, 0, 1, 8, 1, ctypes.cast(shape, ctypes.POINTER(ctypes.c_int64)))


def test_device_count_and_default_pool(native_libs):
    from raf_amd import runtime

    assert runtime.device_count() >= 1
    assert runtime.device_count(runtime.DEV_CPU) >= 1
    runtime.remove_pool()
    name, used, total = runtime.pool_info()
    assert name == "no_pool"  # stream-ordered allocation is available: the cuda >= 11.3 strategy
    assert runtime.alloc_bytes(5) == 5


def test_alloc_and_copies_in_all_directions(native_libs):
    from raf_amd import runtime

    keep = []
    n = 1 << 20
    src = np.random.default_rng(1).integers(0, 256, n, dtype=np.uint8)
    a = runtime.Memory(runtime.DEV_ROCM, 0, n)
    b = runtime.Memory(runtime.DEV_ROCM, 0, n)
    assert a.data and b.data and a.data != b.data and a.data % 256 == 0
    runtime.copy(_host_desc(src, keep), _dev_desc(a.data, n, keep))               # host -> device
    runtime.copy(_dev_desc(a.data, n, keep), _dev_desc(b.data, n, keep))          # device -> device
    back = np.zeros(n, np.uint8)
    runtime.copy(_dev_desc(b.data, n, keep), _host_desc(back, keep))              # device -> host
    assert np.array_equal(back, src)
    other = np.zeros(n, np.uint8)
    runtime.copy(_host_desc(src, keep), _host_desc(other, keep))                  # host -> host
    assert np.array_equal(other, src)
    with pytest.raises(native_libs.RafError, match="sizes differ"):
        runtime.copy(_host_desc(src[:10], keep), _dev_desc(a.data, n, keep))
    a.close()
    b.close()
    assert runtime.Memory(runtime.DEV_ROCM, 0, 0).data is None


def test_streams_events_and_ordering(native_libs):
    from raf_amd import runtime

    keep = []
    n = 64 << 20
    s1, s2 = runtime.Stream(), runtime.Stream()
    assert s1.handle and s2.handle and s1.handle != s2.handle
    e0, e1, e2 = runtime.Event(), runtime.Event(), runtime.Event()
    a = runtime.Memory(runtime.DEV_ROCM, 0, n)
    b = runtime.Memory(runtime.DEV_ROCM, 0, n)
    c = runtime.Memory(runtime.DEV_ROCM, 0, n)
    src = torch.arange(n // 4, dtype=torch.int32).numpy().view(np.uint8)
    runtime.copy(_host_desc(src, keep), _dev_desc(a.data, n, keep))
    e0.record(s1)
    runtime.copy(_dev_desc(a.data, n, keep), _dev_desc(b.data, n, keep), s1)  # on stream 1
    e1.record(s1)
    s2.wait_event(e1)                                                        # stream 2 after stream 1
    runtime.copy(_dev_desc(b.data, n, keep), _dev_desc(c.data, n, keep), s2)
    e2.record(s2)
    e2.synchronize()
    assert e0.elapsed_ms(e1) > 0.0
    back = np.zeros(n, np.uint8)
    runtime.copy(_dev_desc(c.data, n, keep), _host_desc(back, keep))
    assert np.array_equal(back, src)
    s1.synchronize()
    runtime.wait_device()
    for x in (e0, e1, e2, s1, s2, a, b, c):
        x.close()
    with pytest.raises(native_libs.RafError, match="null event"):
        native_libs.check_raf(native_libs.dialect().rafhip_raf_wait(10, 0, 2, None))


def test_stream_ordered_allocation_uses_the_hip_pool(native_libs):
    from raf_amd import runtime

    runtime.remove_pool()
    s = runtime.Stream()
    _, used0, _ = runtime.pool_info()
    chunks = [runtime.Memory(runtime.DEV_ROCM, 0, 8 << 20, 256, s.handle, stream_ordered=True) for _ in range(4)]
    assert len({c.data for c in chunks}) == 4 and all(c.data % 256 == 0 for c in chunks)
    _, used1, total1 = runtime.pool_info()
    assert used1 - used0 == pytest.approx(32.0) and total1 >= used1
    for c in chunks:
        c.close()
    s.synchronize()
    _, used2, total2 = runtime.pool_info()
    assert used2 == pytest.approx(used0) and total2 >= used2  # everything handed back
    again = runtime.Memory(runtime.DEV_ROCM, 0, 8 << 20, 256, s.handle, stream_ordered=True)
    assert again.data and again.data % 256 == 0
    again.close()
    s.synchronize()
    s.close()


def test_page_unit_pool_on_the_device(native_libs):
    from raf_amd import runtime

    runtime.init_pool("page_unit_pool")
    try:
        assert runtime.pool_info()[0] == "page_unit_pool"
        assert runtime.alloc_bytes(1) == 4096 and runtime.alloc_bytes(8193) == 12288
        a = runtime.Memory(runtime.DEV_ROCM, 0, 5000)
        p = a.data
        b = runtime.Memory(runtime.DEV_ROCM, 0, 6000)
        assert b.data != p
        a.close()
        c = runtime.Memory(runtime.DEV_ROCM, 0, 7000)  # same page count: the idle chunk comes back
        assert c.data == p
        with pytest.raises(native_libs.RafError, match="Please use NoPool"):
            runtime.Memory(runtime.DEV_ROCM, 0, 64, 0, None, stream_ordered=True)
        b.close()
        c.close()
        runtime.reset_pool()
        assert runtime.pool_info()[0] == "page_unit_pool"
    finally:
        runtime.init_pool("no_pool")
    assert runtime.pool_info()[0] == "no_pool"


def test_operator_runs_on_a_pool_workspace(native_libs):
    """raf_amd.op.lans takes its workspace from the device's memory pool, stream-ordered."""
    from oracle import lans_f64
    from raf_amd import op, runtime
    from tests.helpers import lans_inputs, max_rel_err

    g, w, m, v = lans_inputs([100, 20000], cfg=300)
    tl = [torch.from_numpy(a).to(DEV) for a in g + w + m + v]
    for step in (1, 2):
        op.lans(tl, torch.tensor(float(step), device=DEV), 1e-3, 0.9, 0.999, 1e-6, True, 0.01, True, True, True)
    ow, om, ov = w, m, v
    for step in (1, 2):
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, lans_f64.LansHParams())
    for t in range(2):
        assert max_rel_err(tl[2 + t].cpu().numpy(), ow[t]) <= 1e-5
    assert runtime.pool_info()[2] > 0.0  # the HIP pool has served the workspaces
