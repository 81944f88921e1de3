"""swiftrt_amd: MI355X-native matmul / Dense path behind SwiftRT's device-queue boundary.

The product is the C-ABI shared library (swiftrt_amd/lib/libSwiftRTHip.so, sources in
swiftrt_amd/csrc, header include/srt_hip.h).  The Python modules here are a thin host-side
mirror of the reference's platform / tensor / operator interface for that path, used to drive
the C ABI from tests and the benchmark.  Importing this package does not load the library;
the first native call does, and raises if it has not been built.
"""
from . import native
from .native import NotSupportedError, SrtError
from .platform import (HipDevice, HipDeviceMemory, HipEvent, HipPlatform, HipQueue, PlanCache, current_queue,
                       using)
from .tensor import (ActivationType, BasicRNNCell, Dense, LSTMCell, Order, Tensor, cast, concatenate, dense_backward,
                     exp, filled, matmul, matmul_gradients, maximum, minimum, relu, sigmoid, tanh)

__all__ = ["native", "NotSupportedError", "SrtError", "HipDevice", "HipDeviceMemory", "HipEvent", "HipPlatform",
           "HipQueue", "current_queue", "using", "ActivationType", "Dense", "Order", "Tensor", "matmul"]
