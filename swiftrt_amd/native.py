"""ctypes binding of the C ABI in include/srt_hip.h (libSwiftRTHip.so).

This is the only place the shared library is loaded.  There is no fallback: if the library
is missing, or a call returns a hard error, an exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SWIFTRT_HIP_LIBRARY selects another build of the same library (e.g. lib/debug/libSwiftRTHip.so from
# `make DEBUG=1`, which checks every launch synchronously)
LIB_PATH = os.environ.get("SWIFTRT_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libSwiftRTHip.so")

# srtStatus
SUCCESS = 0
ERROR_INVALID_VALUE = 1
ERROR_OUT_OF_MEMORY = 2
ERROR_NO_DEVICE = 100
ERROR_NOT_READY = 600
ERROR_LAUNCH_FAILURE = 719
ERROR_NOT_SUPPORTED = 801

# srtDataType
REAL32F, REAL64F, REAL16F, REAL16BF = 0, 1, 2, 14
# srtOrder
ORDER_COL, ORDER_ROW = 0, 1
# srtMemcpyKind
H2D, D2H, D2D = 1, 2, 3


class SrtError(RuntimeError):
    """A hard error reported by the native module (the reference traps on these)."""

    def __init__(self, status, what):
        self.status = status
        super().__init__(f"{what}: {status_string(status)} ({status})")


class NotSupportedError(SrtError):
    """srtErrorNotSupported: the native module asks the caller to use its own CPU path."""


class TensorDescriptor(ctypes.Structure):
    _fields_ = [("type", ctypes.c_int32), ("rank", ctypes.c_uint32), ("order", ctypes.c_int32),
                ("count", ctypes.c_size_t), ("spanCount", ctypes.c_size_t),
                ("shape", ctypes.POINTER(ctypes.c_size_t)), ("strides", ctypes.POINTER(ctypes.c_size_t)),
                ("logicalStrides", ctypes.POINTER(ctypes.c_size_t))]


class DeviceProperties(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 256), ("archName", ctypes.c_char * 64),
                ("totalGlobalMem", ctypes.c_size_t), ("multiProcessorCount", ctypes.c_int32),
                ("clockRateKHz", ctypes.c_int32), ("memoryClockRateKHz", ctypes.c_int32),
                ("memoryBusWidthBits", ctypes.c_int32), ("l2CacheBytes", ctypes.c_int32),
                ("sharedMemPerBlockBytes", ctypes.c_int32), ("warpSize", ctypes.c_int32)]


_vp = ctypes.c_void_p
_i32 = ctypes.c_int32
_descp = ctypes.POINTER(TensorDescriptor)

# name -> (restype, argtypes); every symbol declared in include/srt_hip.h
SIGNATURES = {
    "srtGetStatusString": (ctypes.c_char_p, [_i32]),
    "srtGetVersion": (_i32, []),
    "srtGetDeviceCount": (_i32, [ctypes.POINTER(_i32)]),
    "srtSetDevice": (_i32, [_i32]),
    "srtGetDevice": (_i32, [ctypes.POINTER(_i32)]),
    "srtGetDeviceProperties": (_i32, [ctypes.POINTER(DeviceProperties), _i32]),
    "srtDeviceSynchronize": (_i32, []),
    "srtStreamCreate": (_i32, [ctypes.POINTER(_vp)]),
    "srtStreamDestroy": (_i32, [_vp]),
    "srtStreamSynchronize": (_i32, [_vp]),
    "srtEventCreate": (_i32, [ctypes.POINTER(_vp), _i32]),
    "srtEventDestroy": (_i32, [_vp]),
    "srtEventRecord": (_i32, [_vp, _vp]),
    "srtStreamWaitEvent": (_i32, [_vp, _vp]),
    "srtEventSynchronize": (_i32, [_vp]),
    "srtEventQuery": (_i32, [_vp]),
    "srtEventElapsedTime": (_i32, [ctypes.POINTER(ctypes.c_float), _vp, _vp]),
    "srtDeviceAllocate": (_i32, [ctypes.POINTER(_vp), ctypes.c_size_t, _vp]),
    "srtDeviceFree": (_i32, [_vp]),
    "srtDeviceEmptyCache": (_i32, []),
    "srtHostAllocate": (_i32, [ctypes.POINTER(_vp), ctypes.c_size_t]),
    "srtHostFree": (_i32, [_vp]),
    "srtMemcpyAsync": (_i32, [_vp, _vp, ctypes.c_size_t, _i32, _vp]),
    "srtMemsetAsync": (_i32, [_vp, _i32, ctypes.c_size_t, _vp]),
    "srtMatmul": (_i32, [_vp, _descp, _i32, _vp, _descp, _i32, _vp, _descp, _vp]),
    "srtMatmulBiasActivation": (_i32, [_vp, _descp, _i32, _vp, _descp, _i32, _vp, _descp, _i32,
                                        ctypes.c_double, _vp, _descp, _vp]),
    "srtMatmulQueryKernel": (_i32, [_descp, _i32, _descp, _i32, _descp, _vp, _vp, _vp,
                                     ctypes.c_char_p, ctypes.c_size_t]),
    "srtDelayStream": (_i32, [ctypes.c_double, _vp]),
    "srtActivationBackwardBias": (_i32, [_vp, _descp, _vp, _descp, _i32, ctypes.c_double, _vp, _descp,
                                          _vp, _descp, _vp]),
    "srtActivationBackwardBiasNoAlloc": (_i32, [_vp, _descp, _vp, _descp, _i32, ctypes.c_double, _vp, _descp,
                                                 _vp, _descp, _vp]),
    "srtMatmulTune": (_i32, [_vp, _descp, _i32, _vp, _descp, _i32, _vp, _descp, _i32, ctypes.c_double, _vp, _descp,
                              _vp, ctypes.c_char_p, ctypes.c_size_t]),
    "srtPlanCacheClear": (_i32, []),
    "srtPlanCacheCount": (_i32, [ctypes.POINTER(ctypes.c_size_t)]),
    "srtPlanCacheSave": (_i32, [ctypes.c_char_p]),
    "srtPlanCacheLoad": (_i32, [ctypes.c_char_p]),
    "srtCopyFlat": (_i32, [_i32, _vp, _i32, _vp, ctypes.c_size_t, _vp]),
    "srtFillFlat": (_i32, [_i32, _vp, _vp, ctypes.c_size_t, _vp]),
}
# element-wise neighbours: tensor-tensor, tensor-element and unary forms share three signatures
for _name in ("Add", "Sub", "Mul", "Div", "Max", "Min"):
    SIGNATURES["srt" + _name] = (_i32, [_vp, _descp, _vp, _descp, _vp, _descp, _vp])
    SIGNATURES["srt" + _name + "TE"] = (_i32, [_vp, _descp, _vp, _vp, _descp, _vp])
    SIGNATURES["srt" + _name + "Flat"] = (_i32, [_i32, _vp, _vp, _vp, ctypes.c_size_t, _vp])
    SIGNATURES["srt" + _name + "TEFlat"] = (_i32, [_vp, _i32, _vp, _vp, ctypes.c_size_t, _vp])
for _name in ("Min", "Max"):
    SIGNATURES["srt" + _name + "FlatTE"] = (_i32, [_i32, _vp, _vp, _vp, ctypes.c_size_t, _vp])
for _name in ("Neg", "Exp", "Sigmoid", "Tanh", "Copy"):
    SIGNATURES["srt" + _name] = (_i32, [_vp, _descp, _vp, _descp, _vp])

_lib = None


def lib():
    """The loaded native module.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C swiftrt_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback implementation")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def status_string(status):
    try:
        return lib().srtGetStatusString(int(status)).decode()
    except Exception:  # library not loadable: still give the number a name
        return "srtStatus"


def check(status, what="srt call"):
    """Mirror of cudaCheck / cpuFallback's split: NotSupported is its own exception."""
    if status == SUCCESS:
        return
    if status == ERROR_NOT_SUPPORTED:
        raise NotSupportedError(status, what)
    raise SrtError(status, what)


def make_descriptor(dtype, shape, strides, order):
    """Build an srtTensorDescriptor; returns (descriptor, keepalive) -- keep `keepalive`
    referenced for the duration of the call, like the stack arrays in Tensor.withTensor."""
    rank = len(shape)
    arr_t = ctypes.c_size_t * rank
    shp = arr_t(*[int(s) for s in shape])
    std = arr_t(*[int(s) for s in strides])
    dense = [1] * rank
    for i in range(rank - 2, -1, -1):
        dense[i] = dense[i + 1] * int(shape[i + 1])
    lst = arr_t(*dense)
    count = 1
    span = 1
    for s, st in zip(shape, strides):
        count *= int(s)
        span += (int(s) - 1) * int(st) if int(s) > 0 else 0
    d = TensorDescriptor(int(dtype), rank, int(order), count, span if count else 0,
                         ctypes.cast(shp, ctypes.POINTER(ctypes.c_size_t)),
                         ctypes.cast(std, ctypes.POINTER(ctypes.c_size_t)),
                         ctypes.cast(lst, ctypes.POINTER(ctypes.c_size_t)))
    return d, (shp, std, lst)
