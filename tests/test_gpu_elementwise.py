"""GPU parity tests of the element-wise neighbours of the path (srtAdd ... srtFillFlat) and of
the recurrent cells built from them, through the C ABI, against the CPU oracle.

Bars: +, -, *, /, max, min, neg, copy / conversion and fill are bit-exact (one correctly rounded
fp32 operation and one rounding to the element type on both sides); exp, sigmoid and tanh go
through different libm implementations, so they are held to 2 units in the last place of the
stored type (fp32: 4e-7 relative + 1e-7 absolute).  The LSTM fixtures of the reference's tests are
reproduced to 1e-6, as there.
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
EXACT_BINARY = [("add", "add"), ("sub", "subtract"), ("mul", "mul"), ("div", "div"), ("max", "max"), ("min", "min")]


def rand_storage(g, shape, dt, scale=2.0):
    return H.encode((g.standard_normal(shape) * scale).astype(np.float32), dt)


def close_transcendental(got_st, want_st, dt, floor=1e-7):
    got, want = H.decode(got_st).astype(np.float64), H.decode(want_st).astype(np.float64)
    tol = 2 * (2.0 ** -23 if dt == H.F32 else 2 * H.ULP[dt])
    return np.all(np.abs(got - want) <= tol * np.abs(want) + floor)


# ---- tensor-tensor, dense: the vector path --------------------------------------------------------
@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("op,fn", EXACT_BINARY)
def test_binary_dense_bit_exact(op, fn, dt):
    g = H.rng(11)
    a_st, b_st = rand_storage(g, (257, 384), dt), rand_storage(g, (257, 384), dt)
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    out = srt.Tensor(shape=a.shape, dtype=a.dtype)
    getattr(srt.current_queue(), fn)(a, b, out)
    assert np.array_equal(out.array(), ora.elementwise(op, a_st, b_st))


@pytest.mark.parametrize("dt", DTS)
def test_vector_path_special_values_bit_exact(dt):
    """NaNs, infinities, sums that overflow to infinity, products that land among the subnormals and exact
    ties, scattered over rows that the 16-byte path handles: the 16-bit encoders must agree with the oracle's
    (NaN -> 0x7FFF for bfloat16, round to nearest even) whichever lanes share a vector with a NaN."""
    g = H.rng(21)
    shape = (96, 512)
    a = (g.standard_normal(shape) * 2.0).astype(np.float32)
    b = (g.standard_normal(shape) * 2.0).astype(np.float32)
    big = {H.F32: 3.0e38, H.F16: 60000.0, H.BF16: 3.0e38}[dt]
    tiny = {H.F32: 1.0e-19, H.F16: 2.0e-4, H.BF16: 1.0e-19}[dt]
    where = g.integers(0, 12, shape)
    a[where == 0] = np.nan
    b[where == 1] = np.nan
    a[where == 2] = np.inf
    b[where == 3] = -np.inf
    a[where == 4] = big
    b[where == 4] = big            # the sum overflows
    a[where == 5] = tiny
    b[where == 5] = tiny * 0.37    # the product is a subnormal of the element type (or underflows)
    a[where == 6] = 1.0
    b[where == 6] = {H.F32: 2.0 ** -24, H.F16: 2.0 ** -11, H.BF16: 2.0 ** -8}[dt]   # 1 + half a step: a tie
    a[where == 7] = -0.0
    b[where == 7] = 0.0
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    ta, tb = srt.Tensor(a_st), srt.Tensor(b_st)
    q = srt.current_queue()

    def same(got_st, want_st):
        # bfloat16 has one NaN (0x7FFF); fp32 and fp16 NaNs may differ in sign between host and device
        if dt == H.BF16:
            return np.array_equal(got_st, want_st)
        nan_g, nan_w = np.isnan(H.decode(got_st)), np.isnan(H.decode(want_st))
        return np.array_equal(nan_g, nan_w) and np.array_equal(got_st[~nan_g], want_st[~nan_w])

    for op, fn in EXACT_BINARY:
        out = srt.Tensor(shape=ta.shape, dtype=ta.dtype)
        getattr(q, fn)(ta, tb, out)
        assert same(out.array(), ora.elementwise(op, a_st, b_st)), op
    out = srt.Tensor(shape=ta.shape, dtype=ta.dtype)
    q.neg(ta, out)
    assert same(out.array(), ora.elementwise("neg", a_st))
    # the backward epilogue's dx goes through the same encoder
    dx = srt.Tensor(shape=ta.shape, dtype=ta.dtype)
    db = srt.Tensor(shape=[shape[1]], dtype=ta.dtype)
    q.activation_backward(ta, tb, srt.ActivationType.identity, 0.0, dx, db)
    assert same(dx.array(), ora.elementwise("mul", b_st, H.encode(np.ones(shape, np.float32), dt)))


def test_every_float_converts_to_bfloat16_as_the_reference_codec_does():
    """All 2^32 fp32 bit patterns through the device's fp32 -> bfloat16 copy (the 16-byte path: hardware converter for
    vectors without a NaN, the scalar encoder for the others) against the oracle's restatement of BFloat16.init
    (platform/common/BFloat16.swift:53-80), in 16 slabs of 2^28."""
    q = srt.current_queue()
    n = 1 << 28
    out = srt.Tensor(shape=[n // 4096, 4096], dtype=np.uint16)
    for slab in range(16):
        bits = np.arange(slab * n, (slab + 1) * n, dtype=np.uint64).astype(np.uint32)
        x = bits.view(np.float32).reshape(n // 4096, 4096)
        q.copy(srt.Tensor(x), out)
        want = ora.encode(x, H.BF16)
        assert np.array_equal(out.array(), want), slab


def test_floats_convert_to_float16_as_ieee_does():
    """fp32 -> fp16 copy on the device against numpy's binary16 (round to nearest even, subnormals kept, overflow to
    infinity): every combination of sign, exponent and upper mantissa bits with the thirteen dropped bits at and next to
    the tie (0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF), the same around the ten further bits a subnormal result drops, and
    2^24 random patterns.  NaNs are compared as NaNs (their payloads are not part of the contract)."""
    q = srt.current_queue()
    upper = np.arange(1 << 19, dtype=np.uint32) << 13
    lows = np.array([0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF], np.uint32)
    bits = (upper[:, None] | lows[None, :]).reshape(-1)
    sub = (np.arange(1 << 9, dtype=np.uint32) << 23)[:, None] | np.array(
        [0x7FFFFF, 0x400000, 0x400001, 0x3FFFFF, 0x200000, 0x600000, 0x100000, 0x300000], np.uint32)[None, :]
    bits = np.concatenate([bits, sub.reshape(-1), H.rng(5).integers(0, 1 << 32, 1 << 24, dtype=np.uint64).astype(np.uint32)])
    bits = bits[: bits.size // 4096 * 4096]
    x = bits.view(np.float32).reshape(-1, 4096)
    out = srt.Tensor(shape=list(x.shape), dtype=np.float16)
    q.copy(srt.Tensor(x), out)
    with np.errstate(all="ignore"):
        want = x.astype(np.float16)
    got = out.array()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


@pytest.mark.parametrize("dt", DTS)
def test_binary_odd_sizes_and_misaligned_views(dt):
    """Extents that are not a multiple of the vector width and views that start off a 16-byte
    boundary take the element-at-a-time path of the same kernel."""
    g = H.rng(12)
    a_st, b_st = rand_storage(g, (33, 131), dt), rand_storage(g, (33, 131), dt)
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    assert np.array_equal((a + b).array(), ora.elementwise("add", a_st, b_st))
    av, bv = a[1:30, 3:100], b[2:31, 5:102]
    got = (av * bv).array()
    assert np.array_equal(got, ora.elementwise("mul", a_st[1:30, 3:100], b_st[2:31, 5:102]))


@pytest.mark.parametrize("dt", DTS)
def test_bias_broadcast_add_and_rank3(dt):
    """matmul(x, W) + bias as the reference spells it: the bias is a stride-0 view of the result's
    shape (Tensor(repeating:to:)); also rank 3 and a column broadcast."""
    g = H.rng(13)
    x_st, bias_st = rand_storage(g, (64, 256), dt), rand_storage(g, (256,), dt)
    x, bias = srt.Tensor(x_st), srt.Tensor(bias_st)
    assert np.array_equal((x + bias).array(), ora.elementwise("add", x_st, bias_st))
    col_st = rand_storage(g, (64, 1), dt)
    assert np.array_equal((x * srt.Tensor(col_st)).array(), ora.elementwise("mul", x_st, col_st))
    t3_st, m_st = rand_storage(g, (5, 17, 24), dt), rand_storage(g, (17, 24), dt)
    assert np.array_equal((srt.Tensor(t3_st) - srt.Tensor(m_st)).array(), ora.elementwise("sub", t3_st, m_st))


@pytest.mark.parametrize("dt", DTS)
def test_transposed_and_column_major_operands(dt):
    g = H.rng(14)
    a_st, b_st = rand_storage(g, (40, 72), dt), rand_storage(g, (72, 40), dt)
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    assert np.array_equal((a + b.t).array(), ora.elementwise("add", a_st, np.ascontiguousarray(b_st.T)))
    ac = srt.Tensor(a_st, order=srt.Order.col)
    bc = srt.Tensor(np.ascontiguousarray(b_st.T), order=srt.Order.col)
    assert np.array_equal((ac * bc).array(), ora.elementwise("mul", a_st, np.ascontiguousarray(b_st.T)))


@pytest.mark.parametrize("dt", DTS)
def test_tensor_element_forms(dt):
    g = H.rng(15)
    a_st = rand_storage(g, (19, 200), dt)
    a = srt.Tensor(a_st)
    e = H.encode(np.array([0.75], np.float32), dt)
    assert np.array_equal((a + 0.75).array(), ora.elementwise("add", a_st, e))
    assert np.array_equal((a * 0.75).array(), ora.elementwise("mul", a_st, e))
    assert np.array_equal((a - 0.75).array(), ora.elementwise("sub", a_st, e))
    assert np.array_equal((a / 0.75).array(), ora.elementwise("div", a_st, e))
    zero = H.encode(np.array([0.0], np.float32), dt)
    assert np.array_equal(srt.relu(a).array(), ora.elementwise("max", a_st, zero))
    assert np.array_equal(srt.minimum(a, 0.75).array(), ora.elementwise("min", a_st, e))
    assert np.array_equal((-a).array(), ora.elementwise("neg", a_st))


@pytest.mark.parametrize("dt", DTS)
def test_max_min_nan_rule(dt):
    """max is `a >= b ? a : b` (CpuMath.swift:1197): a NaN on the left yields the right operand,
    a NaN on the right is returned."""
    a_st = H.encode(np.array([[np.nan, 1.0, np.nan, -0.0]], np.float32), dt)
    b_st = H.encode(np.array([[2.0, np.nan, np.nan, 0.0]], np.float32), dt)
    got = H.decode(srt.maximum(srt.Tensor(a_st), srt.Tensor(b_st)).array())
    assert got[0, 0] == 2.0 and np.isnan(got[0, 1]) and np.isnan(got[0, 2])
    assert np.array_equal(srt.maximum(srt.Tensor(a_st), srt.Tensor(b_st)).array()[:, :1],
                          ora.elementwise("max", a_st, b_st)[:, :1])


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("op", ["exp", "sigmoid", "tanh"])
def test_transcendentals(op, dt):
    g = H.rng(16)
    a_st = rand_storage(g, (48, 160), dt, scale=3.0)
    got = getattr(srt, op)(srt.Tensor(a_st)).array()
    assert close_transcendental(got, ora.elementwise(op, a_st), dt)
    # small arguments, where 1 - 2 / (exp(2a) + 1) and 1 / (1 + exp(-a)) - 1/2 lose their digits
    tiny = H.encode((np.logspace(-9, -0.5, 512) * np.where(np.arange(512) % 2, -1.0, 1.0)).astype(np.float32).reshape(8, 64), dt)
    assert close_transcendental(getattr(srt, op)(srt.Tensor(tiny)).array(), ora.elementwise(op, tiny), dt, floor=1e-12)
    # closed forms on exact inputs
    z = H.encode(np.zeros((1, 8), np.float32), dt)
    want = {"exp": 1.0, "sigmoid": 0.5, "tanh": 0.0}[op]
    assert np.all(H.decode(getattr(srt, op)(srt.Tensor(z)).array()) == want)


@pytest.mark.parametrize("src", DTS)
@pytest.mark.parametrize("dst", DTS)
def test_conversion(src, dst):
    """srtCopy between any two of Float / Float16 / BFloat16: round to nearest even, exact when
    widening; bit-exact against the oracle's codecs."""
    g = H.rng(17)
    vals = (g.standard_normal((31, 96)) * 100).astype(np.float32)
    vals[0, :4] = [np.inf, -np.inf, 65519.9, 1e-8]      # fp16 overflow boundary, bf16/fp16 underflow
    a_st = H.encode(vals, src)
    got = srt.cast(srt.Tensor(a_st), H.NP_STORAGE[dst]).array()
    want = ora.elementwise("copy", a_st, out_dtype=dst)
    assert got.dtype == want.dtype and np.array_equal(got, want)


@pytest.mark.parametrize("dt", DTS)
def test_flat_forms_and_fill(dt):
    g = H.rng(18)
    n = 100003
    a_st, b_st = rand_storage(g, (n,), dt), rand_storage(g, (n,), dt)
    q = srt.current_queue()
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    out = srt.Tensor(shape=[n], dtype=a.dtype)
    L = native.lib()
    native.check(L.srtAddFlat(a.type_id, a.device_read(q), b.device_read(q), out.device_read_write(q), n, q.stream))
    assert np.array_equal(out.array(), ora.elementwise("add", a_st, b_st))
    other = H.BF16 if dt != H.BF16 else H.F32
    conv = srt.Tensor(shape=[n], dtype=H.NP_STORAGE[other])
    native.check(L.srtCopyFlat(a.type_id, a.device_read(q), conv.type_id, conv.device_read_write(q), n, q.stream))
    assert np.array_equal(conv.array(), ora.elementwise("copy", a_st, out_dtype=other))
    f = srt.filled([7, 33], -1.5, H.NP_STORAGE[dt])
    assert np.all(H.decode(f.array()) == -1.5)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("op,fn", EXACT_BINARY)
def test_binary_flat_and_element_flat_forms(op, fn, dt):
    """srtXFlat / srtXTEFlat (the reference's srtAddFlat / srtAddTEFlat, math_api.h:81-100, for all six
    operators) called directly on dense buffers whose count is not a multiple of the vector width,
    and the strided forms on the same dense operands: all bit-exact against the oracle."""
    g = H.rng(19)
    n = 70001
    a_st, b_st = rand_storage(g, (n,), dt), rand_storage(g, (n,), dt)
    e = H.encode(np.array([-1.25], np.float32), dt)
    q = srt.current_queue()
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    out = srt.Tensor(shape=[n], dtype=a.dtype)
    L = native.lib()
    name = {"add": "Add", "sub": "Sub", "mul": "Mul", "div": "Div", "max": "Max", "min": "Min"}[op]
    native.check(getattr(L, f"srt{name}Flat")(a.type_id, a.device_read(q), b.device_read(q), out.device_read_write(q),
                                             n, q.stream))
    assert np.array_equal(out.array(), ora.elementwise(op, a_st, b_st))
    native.check(getattr(L, f"srt{name}TEFlat")(a.device_read(q), a.type_id, ctypes.c_void_p(e.ctypes.data),
                                               out.device_read_write(q), n, q.stream))
    assert np.array_equal(out.array(), ora.elementwise(op, a_st, e))
    if op in ("max", "min"):
        native.check(getattr(L, f"srt{name}FlatTE")(a.type_id, a.device_read(q), ctypes.c_void_p(e.ctypes.data),
                                                   out.device_read_write(q), n, q.stream))
        assert np.array_equal(out.array(), ora.elementwise(op, a_st, e))
    # the host mirror takes the Flat forms for dense operands; with them off it takes the strided ones
    q.use_flat_forms = False
    try:
        getattr(q, fn)(a, b, out)
        assert np.array_equal(out.array(), ora.elementwise(op, a_st, b_st))
        getattr(q, fn)(a, -1.25, out)
        assert np.array_equal(out.array(), ora.elementwise(op, a_st, e))
    finally:
        q.use_flat_forms = True
    getattr(q, fn)(a, -1.25, out)
    assert np.array_equal(out.array(), ora.elementwise(op, a_st, e))
    assert getattr(L, f"srt{name}Flat")(native.REAL64F, None, None, None, 4, q.stream) == native.ERROR_NOT_SUPPORTED
    assert getattr(L, f"srt{name}TEFlat")(None, a.type_id, None, None, 4, q.stream) == native.ERROR_INVALID_VALUE
    assert getattr(L, f"srt{name}TEFlat")(None, a.type_id, None, None, 0, q.stream) == native.SUCCESS


def test_errors_and_empty():
    q = srt.current_queue()
    L = native.lib()
    a = srt.Tensor(np.zeros((4, 8), np.float32))
    b = srt.Tensor(np.zeros((4, 9), np.float32))
    out = srt.Tensor(shape=[4, 8], dtype=np.float32)
    ad, k1 = a.descriptor()
    bd, k2 = b.descriptor()
    od, k3 = out.descriptor()
    args = (a.device_read(q), ctypes.byref(ad), b.device_read(q), ctypes.byref(bd), out.device_read_write(q),
            ctypes.byref(od), q.stream)
    assert L.srtAdd(*args) == native.ERROR_INVALID_VALUE            # shapes differ
    ad.type = native.REAL64F
    assert L.srtAdd(a.device_read(q), ctypes.byref(ad), a.device_read(q), ctypes.byref(ad), out.device_read_write(q),
                    ctypes.byref(od), q.stream) == native.ERROR_NOT_SUPPORTED   # caller's CPU fallback
    assert L.srtAdd(None, None, None, None, None, None, q.stream) == native.ERROR_INVALID_VALUE
    e = srt.Tensor(shape=[0, 8], dtype=np.float32)
    assert (e + e).array().shape == (0, 8)
    assert L.srtFillFlat(native.REAL32F, None, None, 0, q.stream) == native.SUCCESS


# ---- the recurrent cells, unfused, on the device ----------------------------------------------------
def test_lstm_fixture_unfused_on_device(kats):
    """LSTMCell as the reference writes it (Recurrent.swift:255-266): concatenate, matmul with bias,
    four gate slices (strided views), sigmoid / tanh, mul, add -- every step a device call --
    reproduces lstmExpectedStates / lstmExpectedOutput to 1e-6 (test_Recurrent.swift:100-167)."""
    k = kats["lstm"]
    cell_layer = srt.LSTMCell(srt.Tensor(np.array(k["lstmInitialCellFusedWeights"], np.float32)),
                              srt.Tensor(np.array(k["lstmInitialCellFusedBias"], np.float32)))
    cell = srt.Tensor(np.array(k["lstmInitialStateCell"], np.float32))
    hidden = srt.Tensor(np.array(k["lstmInitialStateHidden"], np.float32))
    states = []
    for x in k["lstmInputs"]:
        cell, hidden = cell_layer(srt.Tensor(np.array([x], np.float32)), cell, hidden)
        states.append(hidden.array())
    assert np.max(np.abs(np.concatenate(states) - np.array(k["lstmExpectedStates"], np.float32))) <= 1e-6
    assert np.max(np.abs(cell.array() - np.array(k["lstmExpectedOutput"], np.float32))) <= 1e-6


@pytest.mark.parametrize("dt", DTS)
def test_basic_rnn_cell_fused_and_unfused(dt):
    """tanh(matmul([x, h], W) + b) (Recurrent.swift:157-161) as one fused Dense call (one rounding)
    and as the reference's three device operations (a rounding after each): both within the
    roundings they make of the fp64 value -- 1e-5 for fp32; one (fused) or three (unfused) roundings
    of the stored type otherwise."""
    g = H.rng(19)
    x_st, h_st = rand_storage(g, (16, 24), dt, 0.5), rand_storage(g, (16, 40), dt, 0.5)
    w_st, b_st = rand_storage(g, (64, 40), dt, 0.2), rand_storage(g, (40,), dt, 0.2)
    w, b = srt.Tensor(w_st), srt.Tensor(b_st)
    fused = srt.BasicRNNCell(w, b, fused=True)(srt.Tensor(x_st), srt.Tensor(h_st)).array()
    unfused = srt.BasicRNNCell(w, b, fused=False)(srt.Tensor(x_st), srt.Tensor(h_st)).array()
    xin = np.concatenate([H.to64(x_st), H.to64(h_st)], axis=1)
    mm = xin @ H.to64(w_st)
    pre = mm + H.to64(b_st)
    want = np.tanh(pre)
    # a rounding of the product or of the pre-activation moves tanh by at most that rounding (slope <= 1)
    for got, roundings in ((fused, 1), (unfused, 3)):
        err = np.abs(H.to64(got) - want)
        bound = 1e-5 if dt == H.F32 else roundings * H.ULP[dt] * np.maximum(np.abs(mm), np.maximum(np.abs(pre), np.abs(want))) + 1e-6
        assert np.all(err <= bound)


@pytest.mark.parametrize("seed", [31, 32, 33, 34])
def test_random_strided_views_bit_exact_and_inside(seed):
    """Random rank (1-5), extents, storage order (any permutation of the dimensions), padding between rows, start
    offsets, and inputs broadcast along random dimensions; the result is a padded, permuted view inside a buffer full of a
    sentinel.  Every supported case must equal the oracle bit for bit inside the view and leave the rest of the result
    buffer alone; a layout that does not collapse to four dimensions is refused with NotSupported, never miscomputed."""
    from numpy.lib.stride_tricks import as_strided
    g = np.random.default_rng(seed)
    q = srt.current_queue()
    ran = refused = vector = 0

    def layout(shape, inputs, friendly):
        rank = len(shape)
        perm = list(range(rank)) if friendly else list(g.permutation(rank))   # perm[-1] is the innermost dimension in storage
        strides = [0] * rank
        running = 1
        for d in reversed(perm):
            if inputs and shape[d] > 1 and g.random() < 0.25:
                continue                                                   # broadcast: stride 0, takes no storage
            strides[d] = running
            pad = 0 if g.random() < 0.5 else int(g.integers(1, 4)) * (8 if friendly else 1)
            running *= shape[d] + pad
        offset = int(g.integers(0, 4)) * (8 if friendly else 1) + (0 if friendly else int(g.integers(0, 3)))
        size = offset + sum((e - 1) * s for e, s in zip(shape, strides)) + 1
        return offset, strides, size

    for case in range(120):
        dt = DTS[int(g.integers(0, 3))]
        rank = int(g.integers(1, 6))
        friendly = g.random() < 0.5
        shape = [int(g.integers(1, 7)) for _ in range(rank)]
        shape[-1] = int(g.integers(1, 6)) * 8 if friendly else int(g.integers(1, 40))
        if rank > 1:
            shape[int(g.integers(0, rank - 1))] = int(g.integers(1, 40))
        op, fn = EXACT_BINARY[int(g.integers(0, len(EXACT_BINARY)))]
        views, gathered = [], []
        for _ in range(2):
            off, strides, size = layout(shape, True, friendly)
            flat = rand_storage(g, (size + 8,), dt)
            base = srt.Tensor(flat)
            views.append(srt.Tensor(shape=shape, order=base.order, _storage=base.storage, _offset=off, _strides=strides))
            gathered.append(np.ascontiguousarray(as_strided(flat[off:], shape, [s * flat.itemsize for s in strides])))
        off, strides, size = layout(shape, False, friendly)
        sentinel = H.encode(np.full(size + 8, 12345.0, np.float32), dt)
        obase = srt.Tensor(sentinel.copy())
        out = srt.Tensor(shape=shape, order=obase.order, _storage=obase.storage, _offset=off, _strides=strides)
        what = (seed, case, dt, shape, op, [v.strides for v in views], strides, off)
        try:
            getattr(q, fn)(views[0], views[1], out)
        except srt.NotSupportedError:
            refused += 1
            assert rank >= 4, what          # up to three dimensions always collapse to at most four
            continue
        want_flat = sentinel.copy()
        as_strided(want_flat[off:], shape, [s * want_flat.itemsize for s in strides])[...] = ora.elementwise(op, gathered[0], gathered[1])
        got_flat = obase.array()
        assert np.array_equal(got_flat.view(np.uint8), want_flat.view(np.uint8)), what
        ran += 1
        vector += friendly
    assert ran >= 90 and vector >= 30, (ran, refused, vector)
