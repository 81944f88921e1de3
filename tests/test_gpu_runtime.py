"""GPU tests of the device / stream / event / memory entry points of the C ABI."""
import ctypes
import time

import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native
from tests import helpers as H

pytestmark = pytest.mark.gpu


def test_platform_enumerates_gfx950():
    p = srt.HipPlatform.local()
    assert len(p.devices) >= 2 and p.devices[0] is None          # device 0 is the CPU slot
    d = p.devices[1]
    assert b"gfx950" in d.properties.archName
    assert d.properties.warpSize == 64 and d.properties.multiProcessorCount >= 200
    assert len(d.queues) == srt.HipPlatform.accelerator_queue_count
    assert srt.current_queue() is d.queues[0]


def test_memcpy_round_trip_and_memset():
    q = srt.current_queue()
    src = np.arange(100003, dtype=np.uint8)
    mem = q.allocate(src.nbytes)
    q.copy_to_device(src.ctypes.data, mem, src.nbytes)
    dst = np.zeros_like(src)
    q.copy_to_host(mem, dst.ctypes.data, src.nbytes)
    q.wait_for_completion()
    assert np.array_equal(src, dst)
    L = native.lib()
    native.check(L.srtMemsetAsync(ctypes.c_void_p(mem.pointer), 0xAB, 1000, q.stream))
    native.check(L.srtMemsetAsync(ctypes.c_void_p(mem.pointer + 1001), 0x11, 7, q.stream))
    q.copy_to_host(mem, dst.ctypes.data, src.nbytes)
    q.wait_for_completion()
    assert np.all(dst[:1000] == 0xAB) and dst[1000] == src[1000] and np.all(dst[1001:1008] == 0x11)
    assert np.array_equal(dst[1008:], src[1008:])


def test_caching_allocator_reuses_blocks_per_stream():
    q = srt.current_queue()
    native.check(native.lib().srtDeviceEmptyCache())     # start from an empty cache
    m = q.allocate(5000)
    p0 = m.pointer
    del m
    m2 = q.allocate(6000)          # same 8 KiB bin, same stream: handed back at once
    assert m2.pointer == p0
    m3 = q.allocate(6000)
    assert m3.pointer != p0
    assert m2.pointer % 256 == 0 and m3.pointer % 256 == 0
    native.check(native.lib().srtDeviceFree(None))
    assert native.lib().srtDeviceFree(ctypes.c_void_p(12345)) == native.ERROR_INVALID_VALUE
    del m2, m3
    native.check(native.lib().srtDeviceEmptyCache())


def test_caching_allocator_orders_blocks_across_streams():
    """A block freed on one stream goes to another stream only when the work the first stream had
    queued by then has finished; to its own stream it goes back at once."""
    p = srt.HipPlatform.local()
    q0, q1 = p.devices[1].queues[0], p.devices[1].queues[1]
    q0.wait_for_completion()
    q1.wait_for_completion()
    native.check(native.lib().srtDeviceEmptyCache())
    m = q0.allocate(3 << 20)
    p0 = m.pointer
    q0.delay(0.2)                  # q0 is busy: work that may still use the block
    del m                          # freed on q0 while the delay runs
    other = q1.allocate(3 << 20)   # another stream asks for the same bin: must not get the busy block
    assert other.pointer != p0
    same = q0.allocate(3 << 20)    # its own stream gets it back at once (stream order protects it)
    assert same.pointer == p0
    del same
    q0.wait_for_completion()
    # q0 has drained: now the block may move to q1 -- as soon as the event that the first request from
    # q1 records on q0 has been processed, which takes the device a moment even on an idle stream
    for _ in range(200):
        again = q1.allocate(3 << 20)
        if again.pointer == p0:
            break
        del again
        time.sleep(0.005)
    assert again.pointer == p0
    del other, again
    q1.wait_for_completion()
    native.check(native.lib().srtDeviceEmptyCache())


def test_events_delay_and_cross_queue_wait():
    p = srt.HipPlatform.local()
    q0, q1 = p.devices[1].queues[0], p.devices[1].queues[1]
    start = q0.record_event(timing=True)
    q0.delay(0.05)
    done = q0.record_event(timing=True)
    assert not done.occurred                      # srtEventQuery -> not ready while the delay spins
    q1.wait(done)                                 # q1 now ordered after q0's delay
    t0 = time.time()
    q1.wait_for_completion()
    assert done.occurred
    assert done.elapsed_ms_since(start) >= 45.0
    assert time.time() - t0 < 5.0


def test_block_used_on_another_queue_is_not_handed_back_early():
    """A block is reusable at once on the stream it was allocated on.  When its last use was on ANOTHER
    queue, the host object orders that queue's work before the free: the allocating queue, which gets the
    same block straight back, is held until the other queue is through with it."""
    import gc
    p = srt.HipPlatform.local()
    q0, q1 = p.devices[1].queues[0], p.devices[1].queues[1]
    n = 1 << 18
    t = srt.Tensor(np.zeros(n, np.float32))
    t.device_read(q0)                                  # allocated on queue 0
    ptr = t.storage.device.pointer
    q0.wait_for_completion()
    start = q0.record_event(timing=True)
    q1.delay(0.05)                                     # queue 1 is busy ...
    t.device_read_write(q1)                            # ... and is the last user of the block
    del t
    gc.collect()                                       # freed while queue 1 still spins
    u = srt.Tensor(np.ones(n, np.float32))
    u.device_read(q0)                                  # same size class, same stream: the same block
    assert u.storage.device.pointer == ptr
    done = q0.record_event(timing=True)
    done.wait()
    assert done.elapsed_ms_since(start) >= 45.0        # queue 0 waited for queue 1's delay before reusing it
    assert np.array_equal(u.array(), np.ones(n, np.float32))


def test_storage_migration_flags():
    # DiscreteStorage's lazy replica movement: first device read copies host->device, a second does not;
    # reading on the host after a device write copies back once
    a = srt.Tensor(np.ones((4, 4), np.float32))
    q = srt.current_queue()
    a.device_read(q)
    assert a.storage.last_copy == "h2d"
    a.device_read(q)
    assert a.storage.last_copy is None
    c = srt.matmul(a, a)
    assert np.array_equal(c.array(), np.full((4, 4), 4, np.float32)) and c.storage.last_copy == "d2h"
    c.array()
    assert c.storage.last_copy is None


def test_using_queue_scope_and_two_queues():
    p = srt.HipPlatform.local()
    q1 = p.devices[1].queues[1]
    a = srt.Tensor(np.full((8, 8), 2, np.float32))
    with srt.using(q1):
        assert srt.current_queue() is q1
        b = srt.matmul(a, a)
    c = srt.matmul(b, a)           # consumed on queue 0: ordered after queue 1 through an event
    assert np.array_equal(c.array(), np.full((8, 8), 2 * 2 * 8 * 2 * 8, np.float32))


def test_cpp_host_mirror_runs_the_reference_kats():
    """The C++ mirror of the Swift host types (swiftrt_amd/host/srt_host.hpp) over the C ABI."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "host_mirror_test")
    assert os.path.exists(exe), "tests/host_mirror_test is built by __graft_entry__.build()"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all checks passed" in out.stdout


def test_native_module_from_several_threads_each_with_its_own_stream():
    """The native module is entered from several threads at once, each driving a stream of its own through the C ABI
    (the allocator and the plan cache are process globals: platform/cuda/device/CudaDevice.swift:141-160 allocates from
    whichever thread owns the tensor).  Every thread allocates, copies, multiplies shapes whose kernels take
    stream-ordered workspaces (split-K parts, shared tiles, fp32 parts) next to small ones, frees, and repeats; every
    product must be exact and identical from round to round."""
    import ctypes
    import threading
    L = native.lib()
    shapes = [(native.REAL16BF, 512, 1024, 4096), (native.REAL16BF, 3072, 1536, 4096), (native.REAL32F, 512, 2048, 2048),
              (native.REAL16BF, 8, 1000, 520), (native.REAL16F, 200, 264, 72), (native.REAL32F, 64, 64, 64),
              (native.REAL16BF, 1024, 1024, 1024)]
    codec = {native.REAL16BF: H.BF16, native.REAL16F: H.F16, native.REAL32F: H.F32}
    problems = []
    g = H.rng(990)
    for (dt, M, N, K) in shapes:
        a = g.integers(-2, 3, (M, K)).astype(np.float32)
        b = g.integers(-2, 3, (K, N)).astype(np.float32)
        want = H.encode((a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32), codec[dt])
        problems.append((dt, M, N, K, np.ascontiguousarray(H.encode(a, codec[dt])), np.ascontiguousarray(H.encode(b, codec[dt])), want))
    errors = []

    def worker(index):
        try:
            native.check(L.srtSetDevice(0))
            stream = ctypes.c_void_p()
            native.check(L.srtStreamCreate(ctypes.byref(stream)))
            for rnd in range(6):
                for j in range(len(problems)):
                    dt, M, N, K, a_st, b_st, want = problems[(j + index) % len(problems)]
                    ptrs = []
                    for nbytes in (a_st.nbytes, b_st.nbytes, want.nbytes):
                        p = ctypes.c_void_p()
                        native.check(L.srtDeviceAllocate(ctypes.byref(p), nbytes, stream))
                        ptrs.append(p)
                    native.check(L.srtMemcpyAsync(ptrs[0], a_st.ctypes.data_as(ctypes.c_void_p), a_st.nbytes, native.H2D, stream))
                    native.check(L.srtMemcpyAsync(ptrs[1], b_st.ctypes.data_as(ctypes.c_void_p), b_st.nbytes, native.H2D, stream))
                    ad, k1 = native.make_descriptor(dt, (M, K), (K, 1), native.ORDER_ROW)
                    bd, k2 = native.make_descriptor(dt, (K, N), (N, 1), native.ORDER_ROW)
                    od, k3 = native.make_descriptor(dt, (M, N), (N, 1), native.ORDER_ROW)
                    native.check(L.srtMatmul(ptrs[0], ctypes.byref(ad), 0, ptrs[1], ctypes.byref(bd), 0, ptrs[2], ctypes.byref(od), stream))
                    got = np.empty_like(want)
                    native.check(L.srtMemcpyAsync(got.ctypes.data_as(ctypes.c_void_p), ptrs[2], got.nbytes, native.D2H, stream))
                    native.check(L.srtStreamSynchronize(stream))
                    for p in ptrs:
                        native.check(L.srtDeviceFree(p))
                    if not np.array_equal(got.view(np.uint8), want.view(np.uint8)):
                        errors.append((index, rnd, dt, M, N, K))
                        return
            native.check(L.srtStreamSynchronize(stream))
        except Exception as e:   # noqa: BLE001 -- reported by the parent
            errors.append((index, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
