"""The store layer's transfer device with the method names of the reference's
``IDevice`` (ucm/store/device/idevice.h:33-58), bound to the ``ucm_device_*``
entry points of libucm_hip.so.

The reference builds one device object per store instance
(``DeviceFactory::Make(deviceId, bufferSize, bufferNumber)``,
ucm/store/device/cuda/cuda_device.cu:222-227) and then moves blocks through it:
``GetBuffer`` for a pinned staging buffer, ``H2DAsync``/``D2HAsync`` plus
``AppendCallback`` per shard, or ``H2DBatchSync``/``D2HBatchSync`` for arrays of
addresses.  This class is that object for Python callers and tests; native
callers bind the C entry points directly.
"""
from __future__ import annotations

import ctypes as C
from typing import Callable, Dict, List, Optional, Sequence

from .. import _lib


class HipBuffer:
    """A pinned host buffer handed out by ``HipDevice.GetBuffer``; it goes back
    to the pool (or is freed) on ``release`` or when the object is dropped, as
    the reference's shared_ptr deleter does (ibuffered_device.h:52-57)."""

    def __init__(self, device: "HipDevice", ptr: int, size: int):
        self._device, self.ptr, self.size = device, ptr, size

    def view(self) -> C.Array:
        return (C.c_ubyte * self.size).from_address(self.ptr)

    def release(self) -> None:
        if self.ptr and self._device._handle:
            _lib.lib().ucm_device_release_buffer(self._device._handle, self.ptr)
        self.ptr = 0

    def __del__(self):
        self.release()


class HipDevice:
    def __init__(self, device_id: int, buffer_size: int, buffer_number: int):
        self.device_id, self.buffer_size, self.buffer_number = device_id, buffer_size, buffer_number
        self._handle: Optional[C.c_void_p] = None
        self._callbacks: Dict[int, object] = {}
        self._done: List[int] = []  # keys of callbacks that have run (appended on the runtime's thread)
        self._next_cb = 0

    # ---- IDevice ----------------------------------------------------------
    def Setup(self) -> None:
        handle = C.c_void_p()
        _lib.call("ucm_device_create", self.device_id, self.buffer_size, self.buffer_number, C.byref(handle))
        self._handle = handle

    def GetBuffer(self, size: int) -> Optional[HipBuffer]:
        ptr = _lib.lib().ucm_device_get_buffer(self._handle, size)
        return HipBuffer(self, ptr, size) if ptr else None

    def H2DSync(self, dst: int, src: int, count: int) -> None:
        _lib.call("ucm_device_h2d_sync", self._handle, dst, src, count)

    def D2HSync(self, dst: int, src: int, count: int) -> None:
        _lib.call("ucm_device_d2h_sync", self._handle, dst, src, count)

    def H2DAsync(self, dst: int, src: int, count: int) -> None:
        _lib.call("ucm_device_h2d_async", self._handle, dst, src, count)

    def D2HAsync(self, dst: int, src: int, count: int) -> None:
        _lib.call("ucm_device_d2h_async", self._handle, dst, src, count)

    def AppendCallback(self, cb: Callable[[bool], None]) -> None:
        key = self._next_cb
        self._next_cb += 1

        def run(ok: int, _user) -> None:
            try:
                cb(bool(ok))
            finally:
                self._done.append(key)

        thunk = _lib.DEVICE_CALLBACK(run)
        self._callbacks[key] = thunk  # the runtime thread calls it later: keep it alive until then
        self._reap()
        _lib.call("ucm_device_append_callback", self._handle, C.cast(thunk, C.c_void_p), None)

    def Synchronized(self) -> None:
        _lib.call("ucm_device_synchronized", self._handle)
        self._reap()

    def H2DBatchSync(self, d_arr: Sequence[int], h_arr: Sequence[int], count: int) -> None:
        self._batch("ucm_device_h2d_batch_sync", d_arr, h_arr, count)

    def D2HBatchSync(self, h_arr: Sequence[int], d_arr: Sequence[int], count: int) -> None:
        self._batch("ucm_device_d2h_batch_sync", h_arr, d_arr, count)

    # ---- beyond the reference interface ------------------------------------
    @property
    def stream(self) -> int:
        return _lib.lib().ucm_device_stream(self._handle) or 0

    def close(self) -> None:
        if self._handle:
            _lib.lib().ucm_device_destroy(self._handle)  # waits for the stream, so every callback has run
            self._handle = None
            self._callbacks.clear()

    def __del__(self):
        self.close()

    # ---- helpers ----------------------------------------------------------
    def _reap(self) -> None:
        while self._done:
            self._callbacks.pop(self._done.pop(), None)

    def _batch(self, fn: str, dst: Sequence[int], src: Sequence[int], count: int) -> None:
        if len(dst) != len(src):
            raise ValueError(f"{fn}: {len(dst)} destinations for {len(src)} sources")
        n = len(dst)
        _lib.call(fn, self._handle, (C.c_void_p * n)(*dst), (C.c_void_p * n)(*src), n, count)
