"""ctypes front end of the CPU oracle (libsrt_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only the test suite, the smoke check and the benchmark's cpu_baseline leg import this
module; the product package never does.

Arrays travel as numpy arrays whose dtype carries the storage format:
float32 -> Float, float16 -> Float16, uint16 -> BFloat16 bit patterns.
Strides are taken from the numpy array (in elements), so views, transposed views and
column-major buffers are passed exactly as stored, the way the reference passes tensors.
"""
import ctypes
import os
import subprocess

import numpy as np

F32, F16, BF16 = 0, 2, 14                      # same numeric ids as the library's srtDataType
ACC_VALUE, ACC_F32 = 0, 1
SIGMOID, RELU, TANH, CLIPPED_RELU, ELU, IDENTITY = range(6)

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.environ.get("SRT_ORACLE_LIBRARY") or os.path.join(_HERE, "libsrt_oracle.so")
_lib = None


def build():
    """Compile the oracle with its Makefile (gcc)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64p = ctypes.POINTER(ctypes.c_int64)
        vp = ctypes.c_void_p
        L.srt_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.srt_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.srt_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.srt_oracle_bf16_to_f32.restype = ctypes.c_float
        L.srt_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.srt_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.srt_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.srt_oracle_f16_to_f32.restype = ctypes.c_float
        L.srt_oracle_matmul.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                        vp, i64p, i64p, ctypes.c_int,
                                        vp, i64p, i64p, ctypes.c_int,
                                        vp, i64p, i64p]
        L.srt_oracle_matmul.restype = ctypes.c_int
        L.srt_oracle_activation.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_float]
        L.srt_oracle_activation.restype = ctypes.c_float
        L.srt_oracle_dense_forward.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               vp, i64p, i64p, ctypes.c_int,
                                               vp, i64p, i64p, ctypes.c_int,
                                               vp, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                                               vp, i64p, i64p]
        L.srt_oracle_dense_forward.restype = ctypes.c_int
        L.srt_oracle_gemm_f64_rows.argtypes = [ctypes.c_int,
                                               vp, i64p, i64p, ctypes.c_int,
                                               vp, i64p, i64p, ctypes.c_int,
                                               ctypes.c_int64, i64p, vp]
        L.srt_oracle_gemm_f64_rows.restype = ctypes.c_int
        L.srt_oracle_max_threads.restype = ctypes.c_int
        L.srt_oracle_encode.argtypes = [ctypes.c_int, vp, vp, ctypes.c_int64]
        L.srt_oracle_decode.argtypes = [ctypes.c_int, vp, vp, ctypes.c_int64]
        L.srt_oracle_bf16_sweep.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        L.srt_oracle_bf16_sweep.restype = ctypes.c_uint64
        _lib = L
    return _lib


def dtype_id(arr):
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float16:
        return F16
    if arr.dtype == np.uint16:
        return BF16
    raise TypeError(f"unsupported storage dtype {arr.dtype}")


def _i64(vals):
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def _elem_strides(arr):
    return [s // arr.itemsize for s in arr.strides]


def _ptr(arr):
    return ctypes.c_void_p(arr.ctypes.data)


def encode(values_f32, dt):
    """float32 array -> storage array of type dt (F32/F16/BF16) using the oracle's codecs."""
    src = np.ascontiguousarray(values_f32, dtype=np.float32)
    np_dt = {F32: np.float32, F16: np.float16, BF16: np.uint16}[dt]
    dst = np.empty(src.shape, dtype=np_dt)
    lib().srt_oracle_encode(dt, _ptr(src), _ptr(dst), src.size)
    return dst


def decode(stored):
    """storage array -> float32 values using the oracle's codecs."""
    src = np.ascontiguousarray(stored)
    dst = np.empty(src.shape, dtype=np.float32)
    lib().srt_oracle_decode(dtype_id(src), _ptr(src), _ptr(dst), src.size)
    return dst


def matmul(lhs, rhs, transpose_lhs=False, transpose_rhs=False, acc=ACC_VALUE, out=None):
    """Restated cpu_matmul on rank-2 or rank-3 storage arrays (any strides)."""
    dt = dtype_id(lhs)
    assert dtype_id(rhs) == dt and lhs.ndim == rhs.ndim and lhs.ndim in (2, 3)
    ls = list(lhs.shape)
    rs = list(rhs.shape)
    if transpose_lhs:
        ls[-1], ls[-2] = ls[-2], ls[-1]
    if transpose_rhs:
        rs[-1], rs[-2] = rs[-2], rs[-1]
    oshape = ls[:-1] + [rs[-1]]
    if out is None:
        out = np.zeros(oshape, dtype=lhs.dtype)
    rc = lib().srt_oracle_matmul(dt, acc, lhs.ndim,
                                 _ptr(lhs), _i64(lhs.shape), _i64(_elem_strides(lhs)), int(transpose_lhs),
                                 _ptr(rhs), _i64(rhs.shape), _i64(_elem_strides(rhs)), int(transpose_rhs),
                                 _ptr(out), _i64(out.shape), _i64(_elem_strides(out)))
    if rc != 0:
        raise ValueError("matmul inner dimensions must be equal")
    return out


def dense_forward(x, w, bias, activation, coef=0.0, transpose_x=False, transpose_w=False,
                  acc=ACC_F32, fused=True):
    dt = dtype_id(x)
    xs = list(x.shape)
    ws = list(w.shape)
    if transpose_x:
        xs.reverse()
    if transpose_w:
        ws.reverse()
    out = np.zeros((xs[0], ws[1]), dtype=x.dtype)
    bptr = _ptr(bias) if bias is not None else ctypes.c_void_p(0)
    bstride = _elem_strides(bias)[0] if bias is not None else 0
    rc = lib().srt_oracle_dense_forward(dt, acc, int(fused),
                                        _ptr(x), _i64(x.shape), _i64(_elem_strides(x)), int(transpose_x),
                                        _ptr(w), _i64(w.shape), _i64(_elem_strides(w)), int(transpose_w),
                                        bptr, bstride, int(activation), float(coef),
                                        _ptr(out), _i64(out.shape), _i64(_elem_strides(out)))
    if rc != 0:
        raise ValueError("dense forward: extents do not agree")
    return out


def activation(kind, x, coef=0.0):
    f = lib().srt_oracle_activation
    flat = np.asarray(x, dtype=np.float32).ravel()
    return np.array([f(kind, coef, float(v)) for v in flat], dtype=np.float32).reshape(np.shape(x))


def gemm_f64_rows(lhs, rhs, rows=None, transpose_lhs=False, transpose_rhs=False):
    """fp64 grading GEMM for the listed rows (all rows when None); returns float64 [nrows, N]."""
    dt = dtype_id(lhs)
    ls = list(lhs.shape)
    rs = list(rhs.shape)
    if transpose_lhs:
        ls.reverse()
    if transpose_rhs:
        rs.reverse()
    if rows is None:
        nrows, rows_p = ls[0], None
    else:
        rows = np.ascontiguousarray(rows, dtype=np.int64)
        nrows, rows_p = rows.size, rows.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))
    out = np.empty((nrows, rs[1]), dtype=np.float64)
    rc = lib().srt_oracle_gemm_f64_rows(dt,
                                        _ptr(lhs), _i64(lhs.shape), _i64(_elem_strides(lhs)), int(transpose_lhs),
                                        _ptr(rhs), _i64(rhs.shape), _i64(_elem_strides(rhs)), int(transpose_rhs),
                                        nrows, rows_p, _ptr(out))
    if rc != 0:
        raise ValueError(f"gemm_f64_rows failed ({rc})")
    return out


# ---- element-wise neighbours of the path (numpy restatement) ------------------------------------
# The reference's CPU definitions, evaluated in E.Value (= float for Float and BFloat16; for
# Float16 the native half arithmetic of +, -, *, / equals the float operation rounded once, since
# binary32 carries more than twice binary16's precision) and stored with one rounding:
#   add/sub/mul/div  mapOp(lhs, rhs, &out, op)        CpuMath.swift:646-662, :1235-1256
#   max / min        `a >= b ? a : b`, `a <= b ? a : b`   CpuMath.swift:1189-1232
#   neg, exp         CpuMath.swift:1286-1292, :943-949
#   sigmoid          `1 / (1 + exp(-x))`               CpuMath.swift:1369-1377
#   tanh             libm tanh                          CpuMath.swift (cpu_tanh)
# numpy's float32 +, -, *, / are the correctly rounded IEEE operations, i.e. exactly what the C
# restatement of these one-line maps would compute; exp/tanh come from the host libm.
# Pinned by: closed forms on exactly representable inputs, the LSTM fixtures (sigmoid, tanh, mul,
# add chained, tests/golden/reference_kats.json), numpy.float16 as an independent library oracle
# for the half results.  Broadcasting follows numpy (stride-0 views), which is what
# Tensor(repeating:to:) passes to the kernels.
def _max(a, b):
    return np.where(a >= b, a, b)


def _min(a, b):
    return np.where(a <= b, a, b)


ELEMENTWISE = {
    "add": lambda a, b: a + b,
    "sub": lambda a, b: a - b,
    "mul": lambda a, b: a * b,
    "div": lambda a, b: a / b,
    "max": _max,
    "min": _min,
    "neg": lambda a, b: -a,
    "exp": lambda a, b: np.exp(a),
    "sigmoid": lambda a, b: np.float32(1) / (np.float32(1) + np.exp(-a)),
    "tanh": lambda a, b: np.tanh(a),
    "copy": lambda a, b: a,
}


def elementwise(op, a, b=None, out_dtype=None):
    """a, b: storage arrays (b may be None, a storage array broadcastable to a, or one storage
    element); returns the storage array of the result (same format as a unless out_dtype)."""
    dt = dtype_id(a)
    fa = decode(a)
    fb = None
    if b is not None:
        fb = np.broadcast_to(decode(np.asarray(b)), fa.shape)
    with np.errstate(all="ignore"):
        r = ELEMENTWISE[op](fa, fb).astype(np.float32)
    return encode(r, dt if out_dtype is None else out_dtype)


def activation_slope(kind, y, coef=0.0):
    """Derivative of the activation written through its output y (what cudnnActivationBackward
    evaluates for these modes): float32 in, float32 out."""
    y = np.asarray(y, dtype=np.float32)
    one, zero = np.float32(1), np.float32(0)
    if kind == SIGMOID:
        return y * (one - y)
    if kind == RELU:
        return np.where(y > 0, one, zero)
    if kind == TANH:
        return one - y * y
    if kind == CLIPPED_RELU:
        return np.where((y > 0) & (y < np.float32(coef)), one, zero)
    if kind == ELU:
        return np.where(y > 0, one, y + np.float32(coef))
    return np.ones_like(y)


def activation_backward_bias(y, dy, kind, coef=0.0):
    """dx = dy * act'(y) rounded once to the storage type; dbias = column sums of the UNROUNDED
    products, returned as float64 (the grading value) -- the kernel sums them in fp32 in its own
    order and rounds once, so it is compared with a tolerance, or exactly on integer data."""
    dt = dtype_id(y)
    g = decode(dy) * activation_slope(kind, decode(y), coef)
    return encode(g, dt), g.astype(np.float64).sum(axis=0)
