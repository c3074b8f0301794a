"""The store layer's transfer device (ucm_device_* / HipDevice) against the
behaviour of the reference's CudaDevice (ucm/store/device/cuda/cuda_device.cu:107-227
on ucm/store/device/ibuffered_device.h:32-66): pool slots are reused, requests the
pool cannot serve get a buffer of their own, copies are byte-exact in both
directions, a callback runs after the copies queued before it, and the batched
copies move arrays of addresses in one call."""
import ctypes as C
import threading

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def device(ucm):
    from ucm_amd.store.hip_device import HipDevice

    dev = HipDevice(0, 64 * 1024, 4)
    dev.Setup()
    yield dev
    dev.close()


def host_array(buf):
    return np.frombuffer(buf.view(), dtype=np.uint8)


def test_pool_slots_and_fallback(device):
    bufs = [device.GetBuffer(64 * 1024) for _ in range(4)]
    ptrs = sorted(b.ptr for b in bufs)
    assert len(set(ptrs)) == 4
    assert [p - ptrs[0] for p in ptrs] == [i * 64 * 1024 for i in range(4)]  # one contiguous pool
    extra = device.GetBuffer(1024)  # pool exhausted: a buffer of its own
    assert extra is not None and not (ptrs[0] <= extra.ptr < ptrs[0] + 4 * 64 * 1024)
    host_array(extra)[:] = 7  # writable pinned memory
    big = device.GetBuffer(1 << 20)  # larger than a slot: never from the pool
    assert big is not None and not (ptrs[0] <= big.ptr < ptrs[0] + 4 * 64 * 1024)
    released = bufs[2].ptr
    bufs[2].release()
    again = device.GetBuffer(100)
    assert again.ptr == released  # the freed slot is handed out again
    assert device.GetBuffer(0) is None


def test_sync_and_async_copies_with_callback(device):
    rng = np.random.default_rng(5)
    n = 48 * 1024
    src, back = device.GetBuffer(n), device.GetBuffer(n)
    data = rng.integers(0, 256, n, dtype=np.uint8)
    host_array(src)[:] = data
    dev_t = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()

    device.H2DSync(dev_t.data_ptr(), src.ptr, n)
    assert np.array_equal(dev_t.cpu().numpy(), data)
    device.D2HSync(back.ptr, dev_t.data_ptr(), n)
    assert np.array_equal(host_array(back), data)

    # stream-ordered: up, down again into another buffer, then the callback
    data2 = rng.integers(0, 256, n, dtype=np.uint8)
    host_array(src)[:] = data2
    host_array(back)[:] = 0
    seen, fired = [], threading.Event()

    def done(ok):
        seen.append((ok, bytes(host_array(back)[:64])))
        fired.set()

    device.H2DAsync(dev_t.data_ptr(), src.ptr, n)
    device.D2HAsync(back.ptr, dev_t.data_ptr(), n)
    device.AppendCallback(done)
    assert fired.wait(30)
    assert seen == [(True, data2[:64].tobytes())]  # the copies before it had landed
    device.Synchronized()
    assert np.array_equal(host_array(back), data2)
    assert np.array_equal(dev_t.cpu().numpy(), data2)


def test_callbacks_run_in_queue_order(device):
    order, last = [], threading.Event()
    for i in range(5):
        device.AppendCallback(lambda ok, i=i: (order.append(i), last.set() if i == 4 else None))
    assert last.wait(30)
    device.Synchronized()
    assert order == [0, 1, 2, 3, 4]


@pytest.mark.parametrize("number,count", [(1, 16), (7, 4096), (300, 65536), (1000, 48)])
def test_batch_copies(ucm, number, count):
    from ucm_amd.store.hip_device import HipDevice

    dev = HipDevice(0, count, 8)
    dev.Setup()
    try:
        rng = np.random.default_rng(number)
        stage = dev.GetBuffer(number * count)  # larger than a slot for all but the first case: a buffer of its own
        back = dev.GetBuffer(number * count)
        data = rng.integers(0, 256, number * count, dtype=np.uint8)
        host_array(stage)[:] = data
        host_array(back)[:] = 0
        # device blocks scattered over a larger tensor, in a shuffled order
        pool = torch.zeros(2 * number, count, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        slots = rng.permutation(2 * number)[:number]
        d_arr = [pool.data_ptr() + int(s) * count for s in slots]
        dev.H2DBatchSync(d_arr, [stage.ptr + i * count for i in range(number)], count)
        want = np.zeros((2 * number, count), dtype=np.uint8)
        want[slots] = data.reshape(number, count)
        assert np.array_equal(pool.cpu().numpy(), want)
        dev.D2HBatchSync([back.ptr + i * count for i in range(number)], d_arr, count)
        assert np.array_equal(host_array(back), data)
    finally:
        dev.close()


def test_batch_argument_checks(device):
    device.H2DBatchSync([], [], 64)  # empty batch: nothing to do
    with pytest.raises(ValueError):
        device.D2HBatchSync([16, 32], [16], 16)


def test_batch_copies_of_odd_sizes_and_addresses(device):
    """Sizes and addresses that are not multiples of 16 take one runtime copy per pair: same bytes."""
    rng = np.random.default_rng(9)
    number, count = 5, 1000 + 7
    stage, back = device.GetBuffer(number * 1024 + 64), device.GetBuffer(number * 1024 + 64)
    data = rng.integers(0, 256, number * 1024 + 64, dtype=np.uint8)
    host_array(stage)[:] = data
    host_array(back)[:] = 0
    pool = torch.zeros(number * 2048, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    d_arr = [pool.data_ptr() + i * 2048 + 3 for i in range(number)]          # odd device addresses
    device.H2DBatchSync(d_arr, [stage.ptr + i * 1024 + 1 for i in range(number)], count)
    got = pool.cpu().numpy()
    for i in range(number):
        assert np.array_equal(got[i * 2048 + 3 : i * 2048 + 3 + count], data[i * 1024 + 1 : i * 1024 + 1 + count]), i
        assert not got[i * 2048 : i * 2048 + 3].any() and not got[i * 2048 + 3 + count : (i + 1) * 2048].any()
    device.D2HBatchSync([back.ptr + i * 1024 + 5 for i in range(number)], d_arr, count)
    for i in range(number):
        assert np.array_equal(host_array(back)[i * 1024 + 5 : i * 1024 + 5 + count], data[i * 1024 + 1 : i * 1024 + 1 + count]), i


def test_batch_copies_with_pageable_host_memory(device):
    """Aligned addresses in ordinary (pageable) host memory: no kernel may touch them, so the call classifies every
    address on the host and moves such a batch with one runtime copy per pair - same bytes, no launch over memory the
    device cannot reach.  Blocks of the hipBlockStore path (fetch_data / dump_data with raw addresses) go the same way."""
    rng = np.random.default_rng(10)
    number, count = 6, 4096
    raw = np.zeros(number * count + 64, np.uint8)
    start = (-raw.ctypes.data) % 16                                         # a 16-byte aligned window of a numpy array
    host = raw[start : start + number * count]
    assert host.ctypes.data % 16 == 0
    host[:] = rng.integers(0, 256, number * count, dtype=np.uint8)
    pool = torch.zeros(number, count, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    d_arr = [pool.data_ptr() + i * count for i in range(number)]
    device.H2DBatchSync(d_arr, [host.ctypes.data + i * count for i in range(number)], count)
    assert np.array_equal(pool.cpu().numpy().reshape(-1), host)
    back_raw = np.zeros(number * count + 64, np.uint8)
    b0 = (-back_raw.ctypes.data) % 16
    back = back_raw[b0 : b0 + number * count]
    device.D2HBatchSync([back.ctypes.data + i * count for i in range(number)], d_arr, count)
    assert np.array_equal(back, host)
    # a mix: one pinned buffer among pageable ones still works (the whole batch takes the per-pair path)
    pinned = device.GetBuffer(count)
    host_array(pinned)[:] = 9
    mixed = [pinned.ptr] + [host.ctypes.data + i * count for i in range(1, number)]
    device.H2DBatchSync(d_arr, mixed, count)
    got = pool.cpu().numpy()
    assert (got[0] == 9).all() and np.array_equal(got[1:].reshape(-1), host[count:])
    with pytest.raises(Exception):
        device.H2DBatchSync(d_arr, [0] + mixed[1:], count)                  # a null address is refused on the host


def test_device_stream_orders_library_kernels(device):
    """A kernel of the library launched on the device's stream is ordered with its copies."""
    from ucm_amd import _lib

    n = 32 * 1024
    stage = device.GetBuffer(n)
    data = np.random.default_rng(2).integers(0, 256, n, dtype=np.uint8)
    host_array(stage)[:] = data
    a = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    b = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    ptrs = torch.tensor([b.data_ptr(), a.data_ptr()], dtype=torch.int64, device="cuda:0")
    torch.cuda.synchronize()
    device.H2DAsync(a.data_ptr(), stage.ptr, n)
    _lib.call("ucm_copy_batch", ptrs.data_ptr(), ptrs.data_ptr() + 8, 1, n, device.stream)
    device.Synchronized()
    assert np.array_equal(b.cpu().numpy(), data)
