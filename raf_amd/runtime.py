"""Python handles over the host layer's device API and memory pools: the ``rocm`` counterpart of
the reference's CUDA device API (src/device_api/cuda/cuda.cc) and its pool front end
(include/raf/memory_pool.h, src/impl/memory_pool.cc), reached through ``include/rafhip_dialect.h``.

The operator front end (``raf_amd.op``) takes its per-call workspaces from here, the way RAF's
executors take them from ``Memory::Alloc`` around ``OpEnv::Execute``
(src/impl/interpreter.cc:286-291, :322-325).
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int32, c_void_p
from typing import Optional, Tuple

from . import _lib
from ._lib import check_raf

DEV_CPU, DEV_ROCM = 1, 10  # include/raf/device.h:37-50
WAIT_DEVICE, WAIT_STREAM, WAIT_EVENT = 0, 1, 2


class Memory:
    """A chunk from a device's memory pool; released when closed or collected."""

    def __init__(self, device_type: int, device_id: int, nbytes: int, alignment: int = 0,
                 stream: Optional[int] = None, stream_ordered: bool = False):
        self._h = c_void_p(None)
        check_raf(_lib.dialect().rafhip_raf_memory_alloc(device_type, device_id, int(nbytes), int(alignment),
                                                         int(stream_ordered), stream, ctypes.byref(self._h)))
        self.nbytes = int(nbytes)
        self.data = _lib.dialect().rafhip_raf_memory_data(self._h)  # None for a zero-byte chunk

    def close(self):
        if self._h:
            check_raf(_lib.dialect().rafhip_raf_memory_free(self._h))
            self._h = c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass


def device_count(device_type: int = DEV_ROCM) -> int:
    n = c_int32(0)
    check_raf(_lib.dialect().rafhip_raf_device_count(device_type, ctypes.byref(n)))
    return n.value


def pool_info(device_type: int = DEV_ROCM, device_id: int = 0) -> Tuple[str, float, float]:
    """(pool name, used MB, pool MB)."""
    name = ctypes.create_string_buffer(64)
    used, total = c_float(0), c_float(0)
    check_raf(_lib.dialect().rafhip_raf_pool_info(device_type, device_id, name, 64, ctypes.byref(used),
                                                  ctypes.byref(total)))
    return name.value.decode(), used.value, total.value


def init_pool(name: str, device_type: int = DEV_ROCM, device_id: int = 0) -> None:
    check_raf(_lib.dialect().rafhip_raf_pool_init(device_type, device_id, name.encode()))


def remove_pool(device_type: int = DEV_ROCM, device_id: int = 0) -> None:
    check_raf(_lib.dialect().rafhip_raf_pool_remove(device_type, device_id))


def reset_pool(device_type: int = DEV_ROCM, device_id: int = 0) -> None:
    check_raf(_lib.dialect().rafhip_raf_pool_reset(device_type, device_id))


def alloc_bytes(nbytes: int, device_type: int = DEV_ROCM, device_id: int = 0) -> int:
    return _lib.dialect().rafhip_raf_pool_alloc_bytes(device_type, device_id, int(nbytes))


class Stream:
    def __init__(self, device_id: int = 0, device_type: int = DEV_ROCM):
        self.device_type, self.device_id = device_type, device_id
        h = c_void_p(None)
        check_raf(_lib.dialect().rafhip_raf_stream_create(device_type, device_id, ctypes.byref(h)))
        self.handle = h.value

    def wait_event(self, event: "Event") -> None:
        check_raf(_lib.dialect().rafhip_raf_stream_wait_event(self.device_type, self.handle, event.handle))

    def synchronize(self) -> None:
        check_raf(_lib.dialect().rafhip_raf_wait(self.device_type, self.device_id, WAIT_STREAM, self.handle))

    def close(self):
        if self.handle:
            check_raf(_lib.dialect().rafhip_raf_stream_free(self.device_type, self.device_id, self.handle))
            self.handle = None


class Event:
    def __init__(self, device_id: int = 0, flags: int = 0, device_type: int = DEV_ROCM):
        self.device_type, self.device_id = device_type, device_id
        h = c_void_p(None)
        check_raf(_lib.dialect().rafhip_raf_event_create(device_type, device_id, flags, ctypes.byref(h)))
        self.handle = h.value

    def record(self, stream: Optional[Stream] = None) -> None:
        check_raf(_lib.dialect().rafhip_raf_event_record(self.device_type, self.handle,
                                                         stream.handle if stream else None))

    def synchronize(self) -> None:
        check_raf(_lib.dialect().rafhip_raf_wait(self.device_type, self.device_id, WAIT_EVENT, self.handle))

    def elapsed_ms(self, end: "Event") -> float:
        ms = c_float(0)
        check_raf(_lib.dialect().rafhip_raf_event_elapsed_ms(self.device_type, self.handle, end.handle,
                                                             ctypes.byref(ms)))
        return ms.value

    def close(self):
        if self.handle:
            check_raf(_lib.dialect().rafhip_raf_event_free(self.device_type, self.device_id, self.handle))
            self.handle = None


def wait_device(device_id: int = 0, device_type: int = DEV_ROCM) -> None:
    check_raf(_lib.dialect().rafhip_raf_wait(device_type, device_id, WAIT_DEVICE, None))


def copy(src_desc, dst_desc, stream: Optional[Stream] = None) -> None:
    """``DeviceAPI::CopyDataFromTo`` on two ``TensorDesc``s (contiguous, equal byte size)."""
    check_raf(_lib.dialect().rafhip_raf_device_copy(src_desc, dst_desc, stream.handle if stream else None))
