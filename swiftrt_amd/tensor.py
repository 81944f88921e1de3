"""Tensor value type, `matmul` operators and the Dense layer above the HIP queue.

Mirrors, for the matmul path only, Tensor's layout fields (Sources/SwiftRTCore/tensor/
Tensor.swift:26-54), `.t` (tensor/TensorInit.swift:844-890), the matmul operators
(operators/Matmul.swift:29-72) and Dense (Sources/SwiftRTLayers/Dense.swift:21-71).
All arithmetic happens in the native module; this file only carries layout and dispatch.
"""
import enum

import numpy as np

from . import native
from .platform import current_queue


class ActivationType(enum.IntEnum):
    """Case order of ActivationType (platform/common/FunctionProperties.swift:44-51)."""
    sigmoid = 0
    relu = 1
    tanh = 2
    clippedRelu = 3
    elu = 4
    identity = 5


class Order(enum.Enum):
    """Order.row / Order.col (tensor/Tensor.swift:177-236); tiled orders are not part of the path."""
    col = native.ORDER_COL
    row = native.ORDER_ROW


# storage dtype <-> srtDataType.  BFloat16 storage is carried as uint16 bit patterns.
_DTYPES = {np.dtype(np.float32): native.REAL32F, np.dtype(np.float16): native.REAL16F,
           np.dtype(np.uint16): native.REAL16BF}


def strides_for(shape, order):
    """Dense strides (tensor/Shape.swift:274-300): row-major, or column-major in the last two dims."""
    shape = [int(s) for s in shape]
    rank = len(shape)
    st = [1] * rank
    for i in range(rank - 2, -1, -1):
        st[i] = st[i + 1] * shape[i + 1]
    if order == Order.col and rank >= 2:
        st[rank - 2], st[rank - 1] = 1, shape[rank - 2]
    return st


class Tensor:
    """Shape + strides + storage offset over a flat storage buffer with a host replica and a
    lazily created device replica (the role of DiscreteStorage's per-device replicas with
    version-based migration, platform/common/DiscreteStorage.swift:211-381)."""

    class _Storage:
        def __init__(self, host):
            self.host = host            # flat numpy array (authoritative when host_version is newest)
            self.device = None          # HipDeviceMemory
            self.host_version = 0
            self.device_version = -1
            self.last_queue = None
            self.last_copy = None       # "h2d" / "d2h": DiscreteStorage.testLastAccessCopiedDeviceMemory role

    def __init__(self, array=None, shape=None, dtype=None, order=Order.row, _storage=None, _offset=0, _strides=None):
        if _storage is not None:
            self.storage, self.offset = _storage, _offset
            self.shape, self.strides, self.order = tuple(shape), tuple(_strides), order
            return
        if array is not None:
            arr = np.asarray(array)
            if dtype is not None:
                arr = arr.astype(dtype)
            if arr.dtype not in _DTYPES:
                raise TypeError(f"unsupported element storage {arr.dtype}")
            shape = arr.shape
            flat = np.ascontiguousarray(arr).reshape(-1).copy()
            if order == Order.col and arr.ndim >= 2:
                # lay the logical values out column-major in the last two dims
                flat = np.ascontiguousarray(np.swapaxes(arr, -1, -2)).reshape(-1).copy()
        else:
            n = int(np.prod(shape)) if len(shape) else 1
            flat = np.zeros(n, dtype=np.dtype(dtype))
        self.storage = Tensor._Storage(flat)
        self.offset = 0
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(strides_for(self.shape, order))
        self.order = order

    # -- layout ------------------------------------------------------------------------------
    @property
    def dtype(self):
        return self.storage.host.dtype

    @property
    def rank(self):
        return len(self.shape)

    @property
    def count(self):
        return int(np.prod(self.shape)) if self.shape else 1

    @property
    def t(self):
        """Zero-copy transpose of the last two dimensions: swaps extents and strides."""
        sh, st = list(self.shape), list(self.strides)
        sh[-1], sh[-2] = sh[-2], sh[-1]
        st[-1], st[-2] = st[-2], st[-1]
        return Tensor(shape=sh, order=self.order, _storage=self.storage, _offset=self.offset, _strides=st)

    def __getitem__(self, key):
        """Basic slicing -> a view sharing storage (ranges and steps; no integer indexing)."""
        if not isinstance(key, tuple):
            key = (key,)
        key = key + (slice(None),) * (self.rank - len(key))
        off, sh, st = self.offset, [], []
        for k, n, s in zip(key, self.shape, self.strides):
            if not isinstance(k, slice):
                raise TypeError("views are built from slices")
            start, stop, step = k.indices(n)
            if step <= 0:
                raise ValueError("negative steps are not supported")
            off += start * s
            sh.append(max(0, (stop - start + step - 1) // step))
            st.append(s * step)
        return Tensor(shape=sh, order=self.order, _storage=self.storage, _offset=off, _strides=st)

    def descriptor(self):
        return native.make_descriptor(_DTYPES[self.dtype], self.shape, self.strides, self.order.value)

    @property
    def type_id(self):
        return _DTYPES[self.dtype]

    @property
    def is_contiguous(self):
        return tuple(self.strides) == tuple(strides_for(self.shape, self.order))

    def element_storage(self, value):
        """One scalar in this tensor's storage format (a 1-element array): what
        `withUnsafePointer(to: element)` hands to the tensor-element entry points."""
        f = np.array([value], dtype=np.float32)
        if self.dtype == np.dtype(np.uint16):       # BFloat16: round to nearest even, NaN -> 0x7FFF
            u = f.view(np.uint32)
            r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
            r[(u & 0x7FFFFFFF) > 0x7F800000] = 0x7FFF
            return r
        return f.astype(self.dtype)

    @staticmethod
    def repeating(other, shape):
        """Tensor(repeating:to:) (tensor/TensorInit.swift): a zero-copy broadcast view -- `other` is
        aligned to the trailing dimensions of `shape`, every repeated dimension gets stride 0."""
        shape = [int(x) for x in shape]
        lead = len(shape) - other.rank
        if lead < 0:
            raise ValueError("cannot repeat to a lower rank")
        strides = [0] * lead
        for e, st, target in zip(other.shape, other.strides, shape[lead:]):
            if e == target:
                strides.append(st)
            elif e == 1:
                strides.append(0)
            else:
                raise ValueError("shape is not a repetition of the tensor's shape")
        return Tensor(shape=shape, order=other.order, _storage=other.storage, _offset=other.offset, _strides=strides)

    # -- operators (operators/Math.swift, AlgebraicField): thin wrappers over the queue functions ----
    def _binary(self, other, fn_name):
        out = Tensor(shape=self.shape, dtype=self.dtype, order=self.order)
        if isinstance(other, Tensor) and other.shape != self.shape:
            other = Tensor.repeating(other, self.shape)
        getattr(current_queue(), fn_name)(self, other, out)
        return out

    def __add__(self, other): return self._binary(other, "add")
    def __sub__(self, other): return self._binary(other, "subtract")
    def __mul__(self, other): return self._binary(other, "mul")
    def __truediv__(self, other): return self._binary(other, "div")
    __radd__ = __add__
    __rmul__ = __mul__

    def __rsub__(self, other):          # element - tensor = -(tensor - element)
        return -(self - other)

    def __neg__(self):
        out = Tensor(shape=self.shape, dtype=self.dtype, order=self.order)
        current_queue().neg(self, out)
        return out

    # -- storage migration -------------------------------------------------------------------
    def _ensure_device(self, queue):
        s = self.storage
        if s.device is None:
            s.device = queue.allocate(s.host.nbytes)
        if s.last_queue is not None and s.last_queue is not queue:
            queue.wait(s.last_queue.record_event())   # cross-queue sync, DiscreteStorage.swift:271-296
        s.last_queue = queue
        s.device.last_queue = queue

    def device_read(self, queue):
        """Pointer to this view's first element on the queue's device, copying host->device when
        the device replica is stale (Tensor.deviceRead, Tensor.swift:558-582)."""
        s = self.storage
        self._ensure_device(queue)
        s.last_copy = None
        if s.device_version < s.host_version:
            queue.copy_to_device(s.host.ctypes.data, s.device, s.host.nbytes)
            queue.wait_for_completion()      # the pageable host buffer may change after return
            s.device_version = s.host_version
            s.last_copy = "h2d"
        return s.device.pointer + self.offset * s.host.itemsize

    def device_read_write(self, queue):
        ptr = self.device_read(queue)
        s = self.storage
        s.device_version = max(s.device_version, s.host_version) + 1
        return ptr

    def array(self):
        """Logical values as a numpy array in storage dtype, syncing device->host first if the
        device replica is newer (the read() on the app thread, Tensor.swift:546-548)."""
        s = self.storage
        s.last_copy = None
        if s.device is not None and s.device_version > s.host_version:
            q = s.last_queue
            q.copy_to_host(s.device, s.host.ctypes.data, s.host.nbytes)
            q.wait_for_completion()
            s.host_version = s.device_version
            s.last_copy = "d2h"
        item = s.host.itemsize
        return np.lib.stride_tricks.as_strided(s.host[self.offset:], shape=self.shape,
                                               strides=[st * item for st in self.strides]).copy()


def _transposed_shape(shape, transposed):
    sh = list(shape)
    if transposed:
        sh[-1], sh[-2] = sh[-2], sh[-1]
    return sh


def matmul(lhs, rhs, transposed_lhs=False, transposed_rhs=False, bias=None):
    """matmul(_:transposed:_:transposed:) and matmul(_:transposed:_:transposed:bias:)
    (operators/Matmul.swift:29-45, :57-72), rank 2, plus the rank-3 batched form whose queue
    function the reference keeps (CudaMatmul.swift:44-61).  The result is dense, in lhs.order.
    With `bias` the intended semantics are implemented (the reference drops the bias)."""
    if lhs.rank != rhs.rank or lhs.rank not in (2, 3):
        raise ValueError("matmul takes two rank-2 or two rank-3 tensors")
    ls = _transposed_shape(lhs.shape, transposed_lhs)
    rs = _transposed_shape(rhs.shape, transposed_rhs)
    if ls[-1] != rs[-2] or (lhs.rank == 3 and ls[0] != rs[0]):
        raise ValueError("matmul inner dimensions must be equal")
    result = Tensor(shape=ls[:-1] + [rs[-1]], dtype=lhs.dtype, order=lhs.order)
    current_queue().matmul(lhs, transposed_lhs, rhs, transposed_rhs, result, bias=bias)
    return result


class Dense:
    """Dense<S, E> (SwiftRTLayers/Dense.swift:21-71): weight [inputSize, outputSize], bias
    [outputSize], activation.  Forward = activation(matmul(input, weight) + bias), computed by one
    fused native call (the reference's callAsFunction is a stub that returns its input)."""

    def __init__(self, weight, bias=None, activation=ActivationType.identity, relu_ceiling=0.0, elu_alpha=1.0):
        if weight.rank != 2:
            raise ValueError("Dense weight must be rank 2")
        if bias is not None and (bias.rank != 1 or bias.shape[0] != weight.shape[1]):
            raise ValueError("Dense bias must have outputSize elements")
        self.weight, self.bias, self.activation = weight, bias, ActivationType(activation)
        self.coef = relu_ceiling if self.activation == ActivationType.clippedRelu else elu_alpha

    def __call__(self, x):
        if x.rank != 2 or x.shape[1] != self.weight.shape[0]:
            raise ValueError("matmul inner dimensions must be equal")
        result = Tensor(shape=[x.shape[0], self.weight.shape[1]], dtype=x.dtype, order=x.order)
        current_queue().matmul(x, False, self.weight, False, result, bias=self.bias,
                               activation=self.activation, coef=self.coef)
        return result


# ---- element-wise functions (operators/Math.swift; queue functions in CudaMath.swift) -------------
def _unary(x, fn_name):
    out = Tensor(shape=x.shape, dtype=x.dtype, order=x.order)
    getattr(current_queue(), fn_name)(x, out)
    return out


def sigmoid(x): return _unary(x, "sigmoid")
def tanh(x): return _unary(x, "tanh")
def exp(x): return _unary(x, "exp")


def maximum(x, other): return x._binary(other, "max")
def minimum(x, other): return x._binary(other, "min")


def relu(x):
    """max(x, 0) (operators/Math.swift relu): the tensor-element form of max."""
    return maximum(x, 0.0)


def cast(x, dtype):
    """cast(_:elementsTo:): conversion between Float, Float16 and BFloat16 storage on the device."""
    out = Tensor(shape=x.shape, dtype=dtype, order=x.order)
    current_queue().copy(x, out)
    return out


def filled(shape, value, dtype, order=Order.row):
    out = Tensor(shape=shape, dtype=dtype, order=order)
    current_queue().fill(out, value)
    return out


def concatenate(a, b, axis):
    """concatenate(_:_:axis:) of two tensors: two strided device copies into views of the result."""
    if a.rank != b.rank or a.dtype != b.dtype:
        raise ValueError("concatenate: rank and element type must agree")
    shape = list(a.shape)
    shape[axis] += b.shape[axis]
    out = Tensor(shape=shape, dtype=a.dtype, order=a.order)
    lo = [slice(None)] * a.rank
    hi = [slice(None)] * a.rank
    lo[axis] = slice(0, a.shape[axis])
    hi[axis] = slice(a.shape[axis], shape[axis])
    q = current_queue()
    q.copy(a, out[tuple(lo)])
    q.copy(b, out[tuple(hi)])
    return out


# ---- backward of the path ---------------------------------------------------------------------------
def matmul_gradients(out_grad, lhs, transposed_lhs, rhs, transposed_rhs):
    """matmulGradients (differentiable/MathDerivatives.swift:460-482): gradients of
    matmul(lhs, transposed:, rhs, transposed:) as two matmuls with transpose flags, each returned
    in the layout its operand is STORED in.  The (false, false) case is the reference's; for the
    transposed cases the reference's table returns some gradients transposed (its shapes only agree
    for square operands), so the products are written out here:
        C = A  B   : dA = dC B^T      dB = A^T dC
        C = A  B^T : dA = dC B        dB = dC^T A
        C = A^T B  : dA = B dC^T      dB = A dC
        C = A^T B^T: dA = B^T dC^T    dB = dC^T A^T"""
    g = out_grad
    if not transposed_lhs and not transposed_rhs:
        return matmul(g, rhs, False, True), matmul(lhs, g, True, False)
    if not transposed_lhs and transposed_rhs:
        return matmul(g, rhs), matmul(g, lhs, True, False)
    if transposed_lhs and not transposed_rhs:
        return matmul(rhs, g, False, True), matmul(lhs, g)
    return matmul(rhs, g, True, True), matmul(g, lhs, True, True)


def dense_backward(layer, x, y, out_grad):
    """Pullback of Dense.callAsFunction at (x -> y): returns (dx, dweight, dbias).
    dz = out_grad * act'(y) and dbias = column sums of dz come from ONE fused pass
    (HipQueue.activation_backward); dx = dz W^T and dW = x^T dz are matmuls with transpose flags
    (matmulGradients' (false, false) row).  Fills the bias pullbacks the reference leaves as
    fatalError() (MathDerivatives.swift:520-554)."""
    dz = Tensor(shape=y.shape, dtype=y.dtype, order=y.order)
    dbias = Tensor(shape=[y.shape[1]], dtype=y.dtype) if layer.bias is not None else None
    current_queue().activation_backward(y, out_grad, layer.activation, layer.coef, dz, dbias)
    dx, dw = matmul_gradients(dz, x, False, layer.weight, False)
    return dx, dw, dbias


# ---- recurrent cells built from the path (SwiftRTLayers/Recurrent.swift) ---------------------------
class BasicRNNCell:
    """BasicRNNCell (Recurrent.swift:110-161): state' = tanh(matmul([x, h], W) + b).  `fused`
    selects one srtMatmulBiasActivation call; otherwise the reference's three queue operations
    (matmul, add with a broadcast bias, tanh) run unfused on the device."""

    def __init__(self, weight, bias, fused=True):
        self.weight, self.bias, self.fused = weight, bias, fused

    def __call__(self, x, state):
        xin = concatenate(x, state, axis=1)
        if self.fused:
            out = Tensor(shape=[xin.shape[0], self.weight.shape[1]], dtype=xin.dtype)
            current_queue().matmul(xin, False, self.weight, False, out, bias=self.bias,
                                   activation=ActivationType.tanh)
            return out
        return tanh(matmul(xin, self.weight) + self.bias)


class LSTMCell:
    """LSTMCell (Recurrent.swift:165-266): gates = matmul([x, h], fusedWeight, bias: fusedBias) cut
    into input, update, forget, output parts (:176, :190-203); cell' = cell * forget + input *
    update; hidden' = tanh(cell') * output (:255-266)."""

    def __init__(self, fused_weight, fused_bias):
        self.fused_weight, self.fused_bias = fused_weight, fused_bias
        self.hidden_size = fused_weight.shape[1] // 4

    def part(self, i, fused):
        h = self.hidden_size
        return fused[:, i * h:(i + 1) * h]

    def __call__(self, x, cell, hidden):
        gate_input = concatenate(x, hidden, axis=1)
        fused = matmul(gate_input, self.fused_weight, bias=self.fused_bias)
        input_gate = sigmoid(self.part(0, fused))
        update_gate = tanh(self.part(1, fused))
        forget_gate = sigmoid(self.part(2, fused))
        output_gate = sigmoid(self.part(3, fused))
        new_cell = cell * forget_gate + input_gate * update_gate
        new_hidden = tanh(new_cell) * output_gate
        return new_cell, new_hidden
