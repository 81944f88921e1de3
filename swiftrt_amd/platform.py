"""HIP platform: device, queue, event and device-memory types above the C ABI.

Python mirror of the roles the reference's CUDA platform fills
(Sources/SwiftRTCore/platform/cuda/device/CudaPlatform.swift, CudaDevice.swift,
CudaQueue.swift, CudaEvent.swift), used by the tests and the benchmark to drive the C ABI
the way a Swift `HipQueue` would.  It holds no arithmetic: every operation is a native call.
"""
import ctypes
import itertools
import threading

from . import native
from .native import check

_queue_ids = itertools.count(1)


class HipEvent:
    """Role of CudaEvent (CudaEvent.swift:43-75): owns a native event, destroyed with the object."""

    def __init__(self, timing=False):
        h = ctypes.c_void_p()
        check(native.lib().srtEventCreate(ctypes.byref(h), 1 if timing else 0), "srtEventCreate")
        self.handle = h
        self.recorded = False

    def wait(self):
        if self.recorded:
            check(native.lib().srtEventSynchronize(self.handle), "srtEventSynchronize")

    @property
    def occurred(self):
        if not self.recorded:
            return True
        st = native.lib().srtEventQuery(self.handle)
        if st == native.ERROR_NOT_READY:
            return False
        check(st, "srtEventQuery")
        return True

    def elapsed_ms_since(self, start):
        ms = ctypes.c_float()
        check(native.lib().srtEventElapsedTime(ctypes.byref(ms), start.handle, self.handle), "srtEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                native.lib().srtEventDestroy(self.handle)
                self.handle = None
        except Exception:
            pass


class HipDeviceMemory:
    """Role of CudaDeviceMemory (CudaDevice.swift:96-162): the host object owns the pointer and
    frees it when released; byte count padded to a multiple of 32 as the reference does."""

    def __init__(self, device_index, byte_count, queue):
        self.device_index = device_index
        self.byte_count = int(byte_count)
        padded = (self.byte_count + 31) // 32 * 32
        p = ctypes.c_void_p()
        check(native.lib().srtDeviceAllocate(ctypes.byref(p), max(padded, 32), queue.stream), "srtDeviceAllocate")
        self.pointer = p.value
        self.version = -1
        self.name = None
        self.queue = queue          # the allocator hands the block back to this queue's stream at once
        self.last_queue = queue     # the queue that used the block last (kept up to date by the tensor)

    def __del__(self):
        """srtDeviceFree makes the block reusable at once on the stream it was allocated on.  Work that
        another queue still has in flight on it must come first: the allocating stream is made to wait for
        an event recorded on that queue (the contract stated with srtDeviceAllocate in the header)."""
        try:
            if self.pointer:
                if self.last_queue is not None and self.last_queue is not self.queue:
                    self.queue.wait(self.last_queue.record_event())
                native.lib().srtDeviceFree(ctypes.c_void_p(self.pointer))
                self.pointer = None
        except Exception:
            pass


class HipQueue:
    """Role of CudaQueue (CudaQueue.swift:22-196): one non-blocking stream on one device."""

    def __init__(self, device_index, gpu_id, name):
        self.id = next(_queue_ids)
        self.device_index = device_index
        self.gpu_id = gpu_id
        self.name = name
        self.creator_thread = threading.get_ident()
        self.uses_cpu = False
        self.memory_type = "discrete"
        self.mode = "async"
        self.use_flat_forms = True   # dense element-wise operands go through the Flat entry points
        L = native.lib()
        check(L.srtSetDevice(gpu_id), "srtSetDevice")
        s = ctypes.c_void_p()
        check(L.srtStreamCreate(ctypes.byref(s)), "srtStreamCreate")
        self.stream = s

    def select(self):
        check(native.lib().srtSetDevice(self.gpu_id), "srtSetDevice")

    # -- DeviceQueue protocol (platform/common/DeviceQueue.swift:22-82) -----------------------
    def allocate(self, byte_count, heap_index=0):
        self.select()
        return HipDeviceMemory(self.device_index, byte_count, self)

    def copy_to_device(self, host_ptr, dst, byte_count):
        check(native.lib().srtMemcpyAsync(ctypes.c_void_p(dst.pointer), ctypes.c_void_p(host_ptr), byte_count,
                                          native.H2D, self.stream), "srtMemcpyAsync(H2D)")

    def copy_to_host(self, src, host_ptr, byte_count):
        check(native.lib().srtMemcpyAsync(ctypes.c_void_p(host_ptr), ctypes.c_void_p(src.pointer), byte_count,
                                          native.D2H, self.stream), "srtMemcpyAsync(D2H)")

    def copy_async(self, src, dst):
        n = min(src.byte_count, dst.byte_count)
        check(native.lib().srtMemcpyAsync(ctypes.c_void_p(dst.pointer), ctypes.c_void_p(src.pointer), n,
                                          native.D2D, self.stream), "srtMemcpyAsync(D2D)")

    def record_event(self, timing=False):
        ev = HipEvent(timing=timing)
        check(native.lib().srtEventRecord(ev.handle, self.stream), "srtEventRecord")
        ev.recorded = True
        return ev

    def wait(self, event):
        if event.recorded:
            check(native.lib().srtStreamWaitEvent(self.stream, event.handle), "srtStreamWaitEvent")

    def wait_for_completion(self):
        check(native.lib().srtStreamSynchronize(self.stream), "srtStreamSynchronize")

    def delay(self, seconds):
        check(native.lib().srtDelayStream(float(seconds), self.stream), "srtDelayStream")

    # -- the matmul path ---------------------------------------------------------------------
    def matmul(self, lhs, transpose_lhs, rhs, transpose_rhs, result, bias=None, activation=None, coef=0.0):
        """Role of CudaQueue.matmul (platform/cuda/functions/CudaMatmul.swift:25-61), rank 2 and 3.

        Operands are moved to this queue's device if stale (Tensor.device_read, the role of
        Tensor.deviceRead), descriptors are built per call and the native entry point is invoked
        on this queue's stream.  srtErrorNotSupported surfaces as NotSupportedError: a Swift
        caller would run its own cpu_matmul there; this module has no CPU arithmetic."""
        from .tensor import ActivationType
        self.select()
        a_ptr = lhs.device_read(self)
        b_ptr = rhs.device_read(self)
        bias_ptr = bias.device_read(self) if bias is not None else None
        o_ptr = result.device_read_write(self)
        ad, ka = lhs.descriptor()
        bd, kb = rhs.descriptor()
        od, ko = result.descriptor()
        L = native.lib()
        if bias is None and activation in (None, ActivationType.identity):
            st = L.srtMatmul(a_ptr, ctypes.byref(ad), int(transpose_lhs), b_ptr, ctypes.byref(bd), int(transpose_rhs),
                             o_ptr, ctypes.byref(od), self.stream)
        else:
            act = ActivationType.identity if activation is None else activation
            if bias is not None:
                biasd, kbias = bias.descriptor()
                biasd_ref = ctypes.byref(biasd)
            else:
                biasd_ref, kbias = None, None
            st = L.srtMatmulBiasActivation(a_ptr, ctypes.byref(ad), int(transpose_lhs), b_ptr, ctypes.byref(bd),
                                           int(transpose_rhs), bias_ptr, biasd_ref, int(act), float(coef),
                                           o_ptr, ctypes.byref(od), self.stream)
            del kbias
        del ka, kb, ko
        check(st, "srtMatmul")

    def tune_matmul(self, lhs, transpose_lhs, rhs, transpose_rhs, result, bias=None, activation=None, coef=0.0):
        """Role of CudaMatmul2.tune (CudaMatmul.swift:112-120): measures every kernel plan the problem
        qualifies for, records the fastest in the native plan cache (used by every later matmul with
        the same shape, layout class and epilogue) and returns its name.  `result` holds the product."""
        from .tensor import ActivationType
        self.select()
        a_ptr, b_ptr = lhs.device_read(self), rhs.device_read(self)
        bias_ptr = bias.device_read(self) if bias is not None else None
        o_ptr = result.device_read_write(self)
        ad, ka = lhs.descriptor()
        bd, kb = rhs.descriptor()
        od, ko = result.descriptor()
        biasd, kbias = bias.descriptor() if bias is not None else (None, None)
        act = ActivationType.identity if activation is None else activation
        name = ctypes.create_string_buffer(64)
        st = native.lib().srtMatmulTune(a_ptr, ctypes.byref(ad), int(transpose_lhs), b_ptr, ctypes.byref(bd),
                                        int(transpose_rhs), bias_ptr,
                                        ctypes.byref(biasd) if bias is not None else None, int(act), float(coef),
                                        o_ptr, ctypes.byref(od), self.stream, name, 64)
        del ka, kb, ko, kbias
        check(st, "srtMatmulTune")
        return name.value.decode()

    # -- element-wise neighbours of the path ----------------------------------------------------
    def _elementwise(self, name, lhs, rhs, out):
        """Role of CudaQueue.add / mul / max ... (platform/cuda/functions/CudaMath.swift:93-150):
        tensor-tensor form when `rhs` is a tensor, tensor-element form when it is a scalar, unary
        form when it is None.  Inputs must already have the shape of `out` (a broadcast operand is
        a stride-0 view, Tensor.repeating)."""
        self.select()
        L = native.lib()
        a_ptr = lhs.device_read(self)
        # dense operands of one shape take the Flat forms, as CudaQueue does when canFlatten holds
        # (CudaMath.swift:103-113)
        binary = name in ("Add", "Sub", "Mul", "Div", "Max", "Min")
        if binary and self.use_flat_forms and rhs is not None and lhs.is_contiguous and out.is_contiguous \
                and lhs.shape == out.shape and lhs.type_id == out.type_id and lhs.order == out.order:
            if not hasattr(rhs, "device_read"):
                element = lhs.element_storage(rhs)
                o_ptr = out.device_read_write(self)
                check(getattr(L, "srt" + name + "TEFlat")(a_ptr, lhs.type_id, ctypes.c_void_p(element.ctypes.data),
                                                          o_ptr, out.count, self.stream), "srt" + name + "TEFlat")
                return
            if rhs.is_contiguous and rhs.shape == out.shape and rhs.type_id == out.type_id and rhs.order == out.order:
                b_ptr = rhs.device_read(self)
                o_ptr = out.device_read_write(self)
                check(getattr(L, "srt" + name + "Flat")(out.type_id, a_ptr, b_ptr, o_ptr, out.count, self.stream),
                      "srt" + name + "Flat")
                return
        ad, ka = lhs.descriptor()
        if rhs is None:
            o_ptr = out.device_read_write(self)
            od, ko = out.descriptor()
            st = getattr(L, "srt" + name)(a_ptr, ctypes.byref(ad), o_ptr, ctypes.byref(od), self.stream)
        elif hasattr(rhs, "device_read"):
            b_ptr = rhs.device_read(self)
            o_ptr = out.device_read_write(self)
            bd, kb = rhs.descriptor()
            od, ko = out.descriptor()
            st = getattr(L, "srt" + name)(a_ptr, ctypes.byref(ad), b_ptr, ctypes.byref(bd), o_ptr, ctypes.byref(od),
                                          self.stream)
            del kb
        else:
            element = lhs.element_storage(rhs)          # one element in the tensor's storage format
            o_ptr = out.device_read_write(self)
            od, ko = out.descriptor()
            st = getattr(L, "srt" + name + "TE")(a_ptr, ctypes.byref(ad), ctypes.c_void_p(element.ctypes.data),
                                                 o_ptr, ctypes.byref(od), self.stream)
        del ka, ko
        check(st, "srt" + name)

    def add(self, lhs, rhs, out): self._elementwise("Add", lhs, rhs, out)
    def subtract(self, lhs, rhs, out): self._elementwise("Sub", lhs, rhs, out)
    def mul(self, lhs, rhs, out): self._elementwise("Mul", lhs, rhs, out)
    def div(self, lhs, rhs, out): self._elementwise("Div", lhs, rhs, out)
    def max(self, lhs, rhs, out): self._elementwise("Max", lhs, rhs, out)
    def min(self, lhs, rhs, out): self._elementwise("Min", lhs, rhs, out)
    def neg(self, x, out): self._elementwise("Neg", x, None, out)
    def exp(self, x, out): self._elementwise("Exp", x, None, out)
    def sigmoid(self, x, out): self._elementwise("Sigmoid", x, None, out)
    def tanh(self, x, out): self._elementwise("Tanh", x, None, out)

    def copy(self, x, out):
        """Role of CudaQueue.copy / cast: element types may differ (srtCopy converts)."""
        self._elementwise("Copy", x, None, out)

    def fill(self, out, value):
        """Role of CudaQueue.fill(_:with:) (platform/cuda/functions/CudaFill.swift): dense `out`."""
        self.select()
        element = out.element_storage(value)
        if not out.is_contiguous:
            raise native.NotSupportedError(native.ERROR_NOT_SUPPORTED, "fill of a strided view")
        o_ptr = out.device_read_write(self)
        check(native.lib().srtFillFlat(out.type_id, o_ptr, ctypes.c_void_p(element.ctypes.data), out.count,
                                       self.stream), "srtFillFlat")

    def activation_backward(self, y, dy, activation, coef, dx, dbias=None, no_alloc=False):
        """Role of CudaActivation.backward (platform/cuda/layers/CudaActivation.swift:101-127) fused
        with the bias gradient: dx = dy * act'(y), dbias = column sums of dx.  no_alloc: the entry
        point that takes its workspace from a fixed array inside the library (the tensors must then
        already be resident on the device, or the mirror's own staging would allocate)."""
        self.select()
        y_ptr, dy_ptr = y.device_read(self), dy.device_read(self)
        dx_ptr = dx.device_read_write(self)
        yd, k1 = y.descriptor()
        dyd, k2 = dy.descriptor()
        dxd, k3 = dx.descriptor()
        if dbias is not None:
            db_ptr = dbias.device_read_write(self)
            dbd, k4 = dbias.descriptor()
            dbd_ref = ctypes.byref(dbd)
        else:
            db_ptr, dbd_ref, k4 = None, None, None
        name = "srtActivationBackwardBiasNoAlloc" if no_alloc else "srtActivationBackwardBias"
        st = getattr(native.lib(), name)(y_ptr, ctypes.byref(yd), dy_ptr, ctypes.byref(dyd),
                                         int(activation), float(coef), dx_ptr, ctypes.byref(dxd),
                                         db_ptr, dbd_ref, self.stream)
        del k1, k2, k3, k4
        check(st, name)

    def __del__(self):
        try:
            if self.stream:
                native.lib().srtStreamDestroy(self.stream)
                self.stream = None
        except Exception:
            pass


class HipDevice:
    """Role of CudaDevice (CudaDevice.swift:22-94).  Index 0 is reserved for the CPU in the
    reference's numbering; GPU i is device i + 1."""

    def __init__(self, index, queue_count):
        self.index = index
        self.gpu_id = index - 1
        props = native.DeviceProperties()
        check(native.lib().srtGetDeviceProperties(ctypes.byref(props), self.gpu_id), "srtGetDeviceProperties")
        self.properties = props
        self.name = f"gpu:{self.gpu_id}"
        self.memory_type = "discrete"
        self.queues = [HipQueue(index, self.gpu_id, f"{self.name}_q{i}") for i in range(queue_count)]

    def describe(self):
        p = self.properties
        return (f"[type: {p.name.decode()}, arch: {p.archName.decode()}, multiprocessors: {p.multiProcessorCount}, "
                f"memory: {p.totalGlobalMem >> 30} GB, clock: {p.clockRateKHz / 1e6:.2f} GHz]")


class HipPlatform:
    """Role of CudaPlatform (CudaPlatform.swift:22-115): enumerates devices, owns the queue stack."""

    accelerator_queue_count = 2   # CudaPlatform.acceleratorQueueCount, CudaPlatform.swift:39
    _local = None
    _lock = threading.Lock()

    def __init__(self):
        n = ctypes.c_int32()
        check(native.lib().srtGetDeviceCount(ctypes.byref(n)), "srtGetDeviceCount")
        if n.value < 1:
            raise native.SrtError(native.ERROR_NO_DEVICE, "HipPlatform: no GPU visible")
        self.devices = [None] + [HipDevice(i + 1, self.accelerator_queue_count) for i in range(n.value)]
        self.queue_stack = [self.devices[1].queues[0]]   # default queue, CudaPlatform.swift:103-104

    @classmethod
    def local(cls):
        with cls._lock:
            if cls._local is None:
                cls._local = HipPlatform()
            return cls._local

    @property
    def current_queue(self):
        return self.queue_stack[-1]


def current_queue():
    """`currentQueue` (platform/common/Platform.swift:78-80)."""
    return HipPlatform.local().current_queue


class using:
    """`using(queue:)` scope: pushes a queue on the stack for the duration of a with-block."""

    def __init__(self, queue):
        self.queue = queue

    def __enter__(self):
        HipPlatform.local().queue_stack.append(self.queue)
        return self.queue

    def __exit__(self, *exc):
        HipPlatform.local().queue_stack.pop()
        return False


class PlanCache:
    """The native module's process-wide matmul plan cache (role of ExecutionPlanCache,
    platform/common/ExecutionPlanner.swift:20-23): filled by HipQueue.tune_matmul, consulted by every
    matmul, persisted as a small text file."""

    @staticmethod
    def clear():
        check(native.lib().srtPlanCacheClear(), "srtPlanCacheClear")

    @staticmethod
    def count():
        n = ctypes.c_size_t(0)
        check(native.lib().srtPlanCacheCount(ctypes.byref(n)), "srtPlanCacheCount")
        return n.value

    @staticmethod
    def save(path):
        check(native.lib().srtPlanCacheSave(str(path).encode()), "srtPlanCacheSave")

    @staticmethod
    def load(path):
        check(native.lib().srtPlanCacheLoad(str(path).encode()), "srtPlanCacheLoad")
