"""GPU parity tests of the backward of the path: srtActivationBackwardBias (activation gradient
fused with the bias gradient) and the two transposed matmuls of matmulGradients, through the
C ABI, against the CPU oracle and fp64.

Bars: dx is bit-exact against the oracle (two correctly rounded fp32 operations and one rounding
on both sides); dbias is an fp32 sum in the kernel's own fixed order, so it is exact on
integer-valued data and otherwise within one rounding of the stored type plus the fp32 summation
bound of the fp64 column sum; whole Dense backward against fp64 with the matmul tolerances.
"""
import ctypes

import numpy as np
import pytest

import swiftrt_amd as srt
from oracle import srt_oracle as ora
from swiftrt_amd import native
from tests import helpers as H

pytestmark = pytest.mark.gpu

DTS = [H.F32, H.F16, H.BF16]
ACTS = [(srt.ActivationType.sigmoid, 0.0), (srt.ActivationType.relu, 0.0), (srt.ActivationType.tanh, 0.0),
        (srt.ActivationType.clippedRelu, 0.75), (srt.ActivationType.elu, 0.5), (srt.ActivationType.identity, 0.0)]


def forward_output(g, shape, act, coef, dt):
    """A plausible forward output y = act(z) in storage format (so that y lies in the activation's range)."""
    z = (g.standard_normal(shape) * 1.5).astype(np.float32)
    return H.encode(_act_np(int(act), z, coef).astype(np.float32), dt)


def _act_np(kind, z, coef):
    if kind == ora.SIGMOID:
        return 1 / (1 + np.exp(-z))
    if kind == ora.RELU:
        return np.maximum(z, 0)
    if kind == ora.TANH:
        return np.tanh(z)
    if kind == ora.CLIPPED_RELU:
        return np.minimum(np.maximum(z, 0), coef)
    if kind == ora.ELU:
        return np.where(z > 0, z, coef * (np.exp(z) - 1))
    return z


def run_backward(y_st, dy_st, act, coef, want_bias=True):
    y, dy = srt.Tensor(y_st), srt.Tensor(dy_st)
    dx = srt.Tensor(shape=y.shape, dtype=y.dtype)
    db = srt.Tensor(shape=[y.shape[1]], dtype=y.dtype) if want_bias else None
    srt.current_queue().activation_backward(y, dy, act, coef, dx, db)
    return dx.array(), (db.array() if want_bias else None)


def check_dbias(db_st, db64, abs64, m, dt):
    err = np.abs(H.to64(db_st) - db64)
    bound = H.ULP[dt] * np.abs(db64) + (m * 2.0 ** -24 + 2.0 ** -20) * abs64 + 1e-30
    assert np.all(err <= bound), f"bias gradient off by {np.max(err / bound)} x bound"


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("act,coef", ACTS)
def test_activation_backward_bias(act, coef, dt):
    g = H.rng(21)
    m, n = 300, 520                                    # vector path (n % 8 == 0), ragged row chunks
    y_st = forward_output(g, (m, n), act, coef, dt)
    dy_st = H.encode(g.standard_normal((m, n)).astype(np.float32), dt)
    dx, db = run_backward(y_st, dy_st, act, coef)
    want_dx, db64 = ora.activation_backward_bias(y_st, dy_st, int(act), coef)
    assert np.array_equal(dx, want_dx)
    abs64 = np.abs(H.to64(dy_st) * ora.activation_slope(int(act), H.decode(y_st), coef)).sum(axis=0)
    check_dbias(db, db64, abs64, m, dt)


@pytest.mark.parametrize("dt", DTS)
def test_backward_scalar_path_views_and_no_bias(dt):
    """Odd extents and strided views take the element-at-a-time variant; dbias may be omitted."""
    g = H.rng(22)
    act, coef = srt.ActivationType.tanh, 0.0
    y_full = forward_output(g, (70, 123), act, coef, dt)
    dy_full = H.encode(g.standard_normal((70, 123)).astype(np.float32), dt)
    dx, db = run_backward(y_full, dy_full, act, coef)
    want_dx, db64 = ora.activation_backward_bias(y_full, dy_full, int(act), coef)
    assert np.array_equal(dx, want_dx)
    abs64 = np.abs(H.to64(dy_full) * ora.activation_slope(int(act), H.decode(y_full), coef)).sum(axis=0)
    check_dbias(db, db64, abs64, 70, dt)
    # views: rows 3.., columns 5..101 of both inputs, dense result
    y, dy = srt.Tensor(y_full)[3:, 5:101], srt.Tensor(dy_full)[3:, 5:101]
    out = srt.Tensor(shape=y.shape, dtype=y.dtype)
    srt.current_queue().activation_backward(y, dy, act, coef, out, None)
    want, _ = ora.activation_backward_bias(np.ascontiguousarray(y_full[3:, 5:101]),
                                           np.ascontiguousarray(dy_full[3:, 5:101]), int(act), coef)
    assert np.array_equal(out.array(), want)


@pytest.mark.parametrize("dt", DTS)
def test_bias_gradient_exact_on_integers(dt):
    """relu mask times small integers: every partial sum is exactly representable, so the column
    sums are exact whatever the order (sum of at most 4096 values of magnitude <= 2)."""
    g = H.rng(23)
    m, n = 4096, 264
    y_st = H.encode(g.integers(-1, 3, (m, n)).astype(np.float32), dt)     # y > 0 two times in four
    dy_st = H.encode(g.integers(-2, 3, (m, n)).astype(np.float32), dt)
    dx, db = run_backward(y_st, dy_st, srt.ActivationType.relu, 0.0)
    mask = H.decode(y_st) > 0
    want = np.where(mask, H.decode(dy_st), 0).astype(np.float64)
    assert np.array_equal(H.to64(dx), want)
    sums = want.sum(axis=0)
    if dt != H.F32:
        # results beyond the exactly representable integer range of the type round once
        assert np.array_equal(db, H.encode(sums.astype(np.float32), dt))
    else:
        assert np.array_equal(H.to64(db), sums)


def test_slopes_match_numerical_derivative():
    """Pins the closed-form slopes the kernel and the oracle share: central differences of the
    oracle's own forward activation in fp64-stepped fp32."""
    z = np.linspace(-2.0, 2.0, 41).astype(np.float32) + np.float32(0.0123)
    for act, coef in ACTS:
        y = _act_np(int(act), z.astype(np.float64), coef)
        h = 1e-6
        num = (_act_np(int(act), z.astype(np.float64) + h, coef) - _act_np(int(act), z.astype(np.float64) - h, coef)) / (2 * h)
        got = ora.activation_slope(int(act), y.astype(np.float32), coef)
        assert np.max(np.abs(got - num)) < 1e-4, act
        y_st = y.astype(np.float32).reshape(1, -1)
        dx, _ = run_backward(y_st, np.ones_like(y_st), act, coef, want_bias=False)
        assert np.max(np.abs(dx[0] - num)) < 1e-4, act


@pytest.mark.parametrize("dt", DTS)
def test_dense_backward_against_fp64(dt):
    """Whole pullback of Dense: y = relu(x W + b); dz, dbias from the fused pass, dx = dz W^T and
    dW = x^T dz from matmuls with transpose flags; graded against fp64 on the same rounded inputs."""
    g = H.rng(24)
    m, k, n = 192, 160, 264
    x_st = H.encode((g.standard_normal((m, k)) * 0.5).astype(np.float32), dt)
    w_st = H.encode((g.standard_normal((k, n)) * 0.1).astype(np.float32), dt)
    b_st = H.encode((g.standard_normal(n) * 0.1).astype(np.float32), dt)
    dy_st = H.encode(g.standard_normal((m, n)).astype(np.float32), dt)
    layer = srt.Dense(srt.Tensor(w_st), srt.Tensor(b_st), srt.ActivationType.relu)
    x = srt.Tensor(x_st)
    y = layer(x)
    dx, dw, db = srt.dense_backward(layer, x, y, srt.Tensor(dy_st))
    y_st = y.array()
    dz64 = np.where(H.to64(y_st) > 0, H.to64(dy_st), 0.0)
    dz_st = H.encode(dz64.astype(np.float32), dt)             # what the fused pass stores
    assert H.max_norm_rel(H.decode(dx.array()), H.to64(dz_st) @ H.to64(w_st).T) <= H.TOL[dt]
    assert H.max_norm_rel(H.decode(dw.array()), H.to64(x_st).T @ H.to64(dz_st)) <= H.TOL[dt]
    check_dbias(db.array(), dz64.sum(axis=0), np.abs(dz64).sum(axis=0), m, dt)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_gradients_all_layouts(ta, tb):
    """matmulGradients for the four transpose cases: each gradient comes back in the layout its
    operand is stored in; exact on small integers."""
    g = H.rng(25)
    m, k, n = 24, 40, 56
    a64 = g.integers(-3, 4, (k, m) if ta else (m, k)).astype(np.float64)
    b64 = g.integers(-3, 4, (n, k) if tb else (k, n)).astype(np.float64)
    dc64 = g.integers(-2, 3, (m, n)).astype(np.float64)
    a, b, dc = (srt.Tensor(v.astype(np.float32)) for v in (a64, b64, dc64))
    da, db = srt.matmul_gradients(dc, a, ta, b, tb)
    opa = a64.T if ta else a64
    opb = b64.T if tb else b64
    want_da = dc64 @ opb.T          # gradient of op(A)
    want_db = opa.T @ dc64          # gradient of op(B)
    assert np.array_equal(da.array(), (want_da.T if ta else want_da).astype(np.float32))
    assert np.array_equal(db.array(), (want_db.T if tb else want_db).astype(np.float32))


def test_backward_full_size_dense_shape():
    """The Dense benchmark shape, bf16: dx bit-exact, bias gradient within bound."""
    g = H.rng(26)
    m, n = 4096, 11008
    y_st = H.bf16_encode_fast(np.maximum(g.standard_normal((m, n), dtype=np.float32), 0))
    dy_st = H.bf16_encode_fast(g.standard_normal((m, n), dtype=np.float32))
    dx, db = run_backward(y_st, dy_st, srt.ActivationType.relu, 0.0)
    want_dx, db64 = ora.activation_backward_bias(y_st, dy_st, ora.RELU)
    rows = np.arange(0, m, 97)
    assert np.array_equal(dx[rows], want_dx[rows])
    assert np.array_equal(dx, want_dx)
    dz64 = np.where(H.decode(y_st) > 0, H.decode(dy_st), 0).astype(np.float64)
    check_dbias(db, db64, np.abs(dz64).sum(axis=0), m, H.BF16)


def test_backward_errors():
    q = srt.current_queue()
    L = native.lib()
    y = srt.Tensor(np.zeros((4, 8), np.float32))
    bad = srt.Tensor(np.zeros((4, 9), np.float32))
    out = srt.Tensor(shape=[4, 8], dtype=np.float32)
    yd, k1 = y.descriptor()
    bd, k2 = bad.descriptor()
    od, k3 = out.descriptor()
    f = L.srtActivationBackwardBias
    assert f(y.device_read(q), ctypes.byref(yd), bad.device_read(q), ctypes.byref(bd), 1, 0.0,
             out.device_read_write(q), ctypes.byref(od), None, None, q.stream) == native.ERROR_INVALID_VALUE
    assert f(y.device_read(q), ctypes.byref(yd), y.device_read(q), ctypes.byref(yd), 17, 0.0,
             out.device_read_write(q), ctypes.byref(od), None, None, q.stream) == native.ERROR_INVALID_VALUE
    yd.type = native.REAL64F
    assert f(y.device_read(q), ctypes.byref(yd), y.device_read(q), ctypes.byref(yd), 1, 0.0,
             out.device_read_write(q), ctypes.byref(od), None, None, q.stream) == native.ERROR_NOT_SUPPORTED
    assert f(None, None, None, None, 1, 0.0, None, None, None, None, q.stream) == native.ERROR_INVALID_VALUE


@pytest.mark.parametrize("seed", [51, 52, 53])
def test_random_shapes_and_views(seed):
    """Random extents (one row to thousands: one or many row chunks), element types, activations, and y / dy / dx as views
    with padded rows, aligned or unaligned starts, sometimes stored column by column; dx inside a sentinel buffer.  dx must
    be the oracle's bit for bit and stay inside its view; the bias gradient exact on integer data and within its bound
    otherwise."""
    from numpy.lib.stride_tricks import as_strided
    g = np.random.default_rng(seed)
    q = srt.current_queue()

    def place(values, aligned, allow_columns):
        m, n = values.shape
        vdt = H.F32 if values.dtype == np.float32 else H.F16 if values.dtype == np.float16 else H.BF16
        unit = 8 if aligned else 1
        by_columns = allow_columns and g.random() < 0.2
        lead, other = (m, n) if by_columns else (n, m)
        pitch = lead + int(g.choice([0, 0, 8, 16] if aligned else [0, 1, 5, 8]))
        off = int(g.integers(0, 4)) * unit
        flat = H.encode(np.full(off + pitch * other + 8, 99.0, np.float32), vdt)
        strides = [1, pitch] if by_columns else [pitch, 1]
        as_strided(flat[off:], (m, n), [s * flat.itemsize for s in strides])[...] = values
        base = srt.Tensor(flat)
        return base, srt.Tensor(shape=[m, n], order=base.order, _storage=base.storage, _offset=off, _strides=strides), flat, off, strides

    for case in range(60):
        dt = DTS[int(g.integers(0, 3))]
        act, coef = ACTS[int(g.integers(0, len(ACTS)))]
        m = int(np.exp(g.uniform(0, np.log(5000))))
        n = int(np.exp(g.uniform(0, np.log(3000))))
        aligned = g.random() < 0.6
        if aligned:
            n = max(8, n // 8 * 8)
        integers = g.random() < 0.4
        if integers:
            act, coef = srt.ActivationType.relu, 0.0
            y_st = H.encode(g.integers(-1, 3, (m, n)).astype(np.float32), dt)
            dy_st = H.encode(g.integers(-2, 3, (m, n)).astype(np.float32), dt)
        else:
            y_st = forward_output(g, (m, n), act, coef, dt)
            dy_st = H.encode(g.standard_normal((m, n)).astype(np.float32), dt)
        _, y, _, _, _ = place(y_st, aligned, True)
        _, dy, _, _, _ = place(dy_st, aligned, True)
        obase, dx, oflat, off, strides = place(np.zeros_like(y_st), aligned, False)
        want_bias = g.random() < 0.8
        db = srt.Tensor(shape=[n], dtype=y.dtype) if want_bias else None
        what = (seed, case, dt, act, m, n, aligned, integers, y.strides, dy.strides, strides, off)
        q.activation_backward(y, dy, act, coef, dx, db)
        want_dx, db64 = ora.activation_backward_bias(y_st, dy_st, int(act), coef)
        want_flat = oflat.copy()
        as_strided(want_flat[off:], (m, n), [s * want_flat.itemsize for s in strides])[...] = want_dx
        assert np.array_equal(obase.array().view(np.uint8), want_flat.view(np.uint8)), what
        if want_bias:
            if integers:
                sums = H.to64(want_dx).sum(axis=0)
                assert np.array_equal(db.array().view(np.uint8), H.encode(sums.astype(np.float32), dt).view(np.uint8)), what
            else:
                abs64 = np.abs(H.to64(dy_st) * ora.activation_slope(int(act), H.decode(y_st), coef)).sum(axis=0)
                check_dbias(db.array(), db64, abs64, m, dt)
