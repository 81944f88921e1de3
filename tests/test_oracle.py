"""Pins the CPU oracle: reference known-answer tests, library oracles, closed forms.

Each check is chosen so that a plausible mistake in the restatement (dropped term, wrong
stride after a transpose, wrong rounding rule, wrong gate order) fails it.
"""
import numpy as np
import pytest

from oracle import srt_oracle as ora


def test_matmul_kat_f32(kats):
    k = kats["matmul_2d"]
    a = np.array(k["a"], dtype=np.float32)
    b = np.array(k["b"], dtype=np.float32)
    c = ora.matmul(a, b)
    assert np.array_equal(c, np.array(k["c"], dtype=np.float32))


def test_matmul_kat_gradients_exercise_transposes(kats):
    # matmulGradients, NN case (differentiable/MathDerivatives.swift:467-470):
    #   dA = matmul(dC, transposed: false, B, transposed: true); dB = matmul(A, transposed: true, dC)
    k = kats["matmul_2d"]
    a = np.array(k["a"], dtype=np.float32)
    b = np.array(k["b"], dtype=np.float32)
    ones = np.ones((3, 4), dtype=np.float32)
    assert np.array_equal(ora.matmul(ones, b, transpose_rhs=True), np.array(k["grad_a_for_ones"], np.float32))
    assert np.array_equal(ora.matmul(a, ones, transpose_lhs=True), np.array(k["grad_b_for_ones"], np.float32))
    # TT case of the table: matmul(B^T stored, T, A^T stored, T) == (A.B)^T ... and
    # matmul(A^T stored, T, B) == A.B
    at = np.ascontiguousarray(a.T)
    bt = np.ascontiguousarray(b.T)
    c = np.array(k["c"], np.float32)
    assert np.array_equal(ora.matmul(at, b, transpose_lhs=True), c)
    assert np.array_equal(ora.matmul(a, bt, transpose_rhs=True), c)
    assert np.array_equal(ora.matmul(at, bt, transpose_lhs=True, transpose_rhs=True), c)
    assert np.array_equal(ora.matmul(b, a, transpose_lhs=True, transpose_rhs=True), c.T)


@pytest.mark.parametrize("np_dt", [np.float32, np.float16, "bf16"])
def test_matmul_batched_kat(kats, np_dt):
    k = kats["matmul_batched"]
    a = np.arange(12, dtype=np.float32).reshape(k["a_arange_shape"])
    b = np.arange(16, dtype=np.float32).reshape(k["b_arange_shape"])
    want = np.array(k["c"], dtype=np.float32)
    if np_dt == "bf16":
        a, b = ora.encode(a, ora.BF16), ora.encode(b, ora.BF16)
    else:
        a, b = a.astype(np_dt), b.astype(np_dt)
    c = ora.matmul(a, b)
    got = ora.decode(c) if np_dt == "bf16" else c.astype(np.float32)
    # values up to 275: exact in fp16, and in bf16 only up to 256 -> compare through the codec
    if np_dt == "bf16":
        assert np.array_equal(got, ora.decode(ora.encode(want, ora.BF16)))
    else:
        assert np.array_equal(got, want)
    # batched gradients: dA = dC . B^T, dB = A^T . dC per batch (transpose swaps last two dims only)
    ones = np.ones((2, 3, 4), dtype=np.float32)
    a32 = np.arange(12, dtype=np.float32).reshape(2, 3, 2)
    b32 = np.arange(16, dtype=np.float32).reshape(2, 2, 4)
    assert np.array_equal(ora.matmul(ones, b32, transpose_rhs=True), np.array(k["grad_a_for_ones"], np.float32))
    assert np.array_equal(ora.matmul(a32, ones, transpose_lhs=True), np.array(k["grad_b_for_ones"], np.float32))


def test_right_batched_kat_via_broadcast_stride(kats):
    k = kats["matmul_right_batched"]
    a = np.arange(6, dtype=np.float32).reshape(3, 2)
    b = np.arange(16, dtype=np.float32).reshape(2, 2, 4)
    a3 = np.broadcast_to(a, (2, 3, 2))  # batch stride 0
    assert np.array_equal(ora.matmul(a3, b), np.array(k["c"], np.float32))


def test_batched_equals_loop_of_single():
    rng = np.random.default_rng(5)
    a = rng.standard_normal((3, 5, 7), dtype=np.float32)
    b = rng.standard_normal((3, 4, 7), dtype=np.float32)
    c = ora.matmul(a, b, transpose_rhs=True)
    for n in range(3):
        assert np.array_equal(c[n], ora.matmul(a[n], b[n], transpose_rhs=True))


def test_sequential_k_order_and_no_fma():
    # k ascending, multiply then add, float accumulator: reproduce with numpy float32 scalars
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (4, 37)).astype(np.float32)
    b = rng.uniform(-1, 1, (37, 3)).astype(np.float32)
    c = ora.matmul(a, b)
    for r in range(4):
        for col in range(3):
            acc = np.float32(0)
            for kk in range(37):
                acc = np.float32(acc + np.float32(a[r, kk] * b[kk, col]))
            assert c[r, col] == acc
    # a case where a fused multiply-add would differ from multiply-then-add
    x = np.float32(1 + 2**-12)
    aa = np.array([[x, 1.0]], dtype=np.float32)
    bb = np.array([[x], [-(1 + 2**-11)]], dtype=np.float32)
    want = np.float32(np.float32(x * x) - np.float32(1 + 2**-11))
    assert ora.matmul(aa, bb)[0, 0] == want == 0.0  # fma would give 2^-24


def test_strided_views_and_column_major():
    rng = np.random.default_rng(2)
    big_a = rng.integers(-8, 9, (10, 12)).astype(np.float32)
    big_b = rng.integers(-8, 9, (12, 14)).astype(np.float32)
    a = big_a[1:8:2, 2:11:3]      # 4 x 3, both strides non-unit
    b = big_b[3:6, 1:13:4]        # 3 x 3
    assert np.array_equal(ora.matmul(a, b), (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32))
    af = np.asfortranarray(big_a)  # column-major storage, strides (1, M)
    out = np.zeros((10, 14), dtype=np.float32, order="F")
    ora.matmul(af, big_b, out=out)
    assert np.array_equal(out, big_a @ big_b)


@pytest.mark.parametrize("dt", [ora.F32, ora.F16, ora.BF16])
def test_integer_inputs_exact_any_order(dt):
    rng = np.random.default_rng(3)
    # |x| <= 8, K = 16 -> |sum| <= 1024 and every partial sum is an integer < 2^11: exact in fp16;
    # bf16 stores 8 bits, so compare through its codec
    a = rng.integers(-8, 9, (9, 16)).astype(np.float32)
    b = rng.integers(-8, 9, (16, 11)).astype(np.float32)
    c = ora.matmul(ora.encode(a, dt), ora.encode(b, dt))
    want = ora.encode((a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32), dt)
    assert np.array_equal(c.view(np.uint16) if dt != ora.F32 else c, want.view(np.uint16) if dt != ora.F32 else want)


def test_ones_and_identity():
    a = np.ones((5, 33), np.float32)
    b = np.ones((33, 6), np.float32)
    assert np.all(ora.matmul(a, b) == 33)
    rng = np.random.default_rng(4)
    m = rng.standard_normal((7, 7), dtype=np.float32)
    assert np.array_equal(ora.matmul(m, np.eye(7, dtype=np.float32)), m)


def test_shape_mismatch_raises():
    with pytest.raises(ValueError):
        ora.matmul(np.zeros((3, 2), np.float32), np.zeros((3, 4), np.float32))


def test_bf16_codec_exhaustive_vs_independent_formula():
    L = ora.lib()
    assert L.srt_oracle_bf16_sweep(0, 0xFFFFFFFF) == 0


def test_bf16_codec_special_cases():
    L = ora.lib()
    f = L.srt_oracle_f32_to_bf16
    assert f(1.0) == 0x3F80
    assert f(np.float32(1.0 + 2**-8)) == 0x3F80          # tie -> even (down)
    assert f(np.float32(1.0 + 3 * 2**-8)) == 0x3F82      # tie -> even (up)
    assert f(np.float32(1.0 + 2**-8 + 2**-20)) == 0x3F81  # above the tie
    assert f(float("nan")) == 0x7FFF
    assert f(float("inf")) == 0x7F80 and f(float("-inf")) == 0xFF80
    assert f(np.float32(3.3895314e38)) == 0x7F7F and f(np.float32(3.4028235e38)) == 0x7F80  # max float rounds up into inf, as RNE does
    assert L.srt_oracle_bf16_to_f32(0x3F80) == 1.0 and L.srt_oracle_bf16_to_f32(0xC000) == -2.0


def test_bf16_add_kat(kats):
    # test_addBFloat16: arange(6) + arange(6) == [0,2,4,6,8,10] through the codec
    a = ora.decode(ora.encode(np.arange(6, dtype=np.float32), ora.BF16))
    assert np.array_equal(ora.decode(ora.encode(a + a, ora.BF16)), np.arange(6, dtype=np.float32) * 2)


def test_f16_codec_vs_numpy():
    L = ora.lib()
    allbits = np.arange(65536, dtype=np.uint16)
    got = ora.decode(allbits.view(np.float16))
    want = allbits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32),
        # exact ties between neighbouring halves, normal and subnormal
        ((allbits[:0x7BFF].view(np.float16).astype(np.float64) + allbits[1:0x7C00].view(np.float16).astype(np.float64)) / 2).astype(np.float32),
        np.array([65504, 65519.99, 65520, 1e9, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001, 0.0, -0.0, np.inf, -np.inf], np.float32),
    ])
    vals = np.concatenate([vals, -vals])
    got = ora.encode(vals, ora.F16).view(np.uint16)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_f16_value_accumulation_matches_numpy_half_arithmetic():
    rng = np.random.default_rng(8)
    a = (rng.standard_normal((3, 50)) * 0.1).astype(np.float16)
    b = (rng.standard_normal((50, 2)) * 0.1).astype(np.float16)
    c = ora.matmul(a, b, acc=ora.ACC_VALUE)
    for r in range(3):
        for col in range(2):
            acc = np.float16(0)
            for kk in range(50):
                acc = np.float16(acc + np.float16(a[r, kk] * b[kk, col]))
            assert c[r, col] == acc
    c32 = ora.matmul(a, b, acc=ora.ACC_F32)
    ref = (a.astype(np.float64) @ b.astype(np.float64))
    assert np.max(np.abs(c32.astype(np.float64) - ref)) <= np.max(np.abs(c.astype(np.float64) - ref)) + 1e-3


def test_gemm_f64_vs_numpy():
    rng = np.random.default_rng(9)
    a = rng.standard_normal((23, 31)).astype(np.float32)
    b = rng.standard_normal((17, 31)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    got = ora.gemm_f64_rows(a, b, transpose_rhs=True)
    assert np.allclose(got, want, rtol=1e-13, atol=1e-13)
    rows = np.array([22, 0, 5])
    assert np.allclose(ora.gemm_f64_rows(a, b, rows=rows, transpose_rhs=True), want[rows], rtol=1e-13, atol=1e-13)
    at = np.ascontiguousarray(a.T)
    assert np.allclose(ora.gemm_f64_rows(at, b, transpose_lhs=True, transpose_rhs=True), want, rtol=1e-13, atol=1e-13)
    ab = ora.encode(a, ora.BF16)
    assert np.allclose(ora.gemm_f64_rows(ab, ora.encode(b, ora.BF16), transpose_rhs=True),
                       ora.decode(ab).astype(np.float64) @ ora.decode(ora.encode(b, ora.BF16)).astype(np.float64).T,
                       rtol=1e-13, atol=1e-13)


def _lstm_run(kats, fused):
    k = kats["lstm"]
    w = np.array(k["lstmInitialCellFusedWeights"], np.float32)       # [8, 16]
    bias = np.array(k["lstmInitialCellFusedBias"], np.float32)        # [16]
    cell = np.array(k["lstmInitialStateCell"], np.float32)
    hidden = np.array(k["lstmInitialStateHidden"], np.float32)
    states = []
    for x in k["lstmInputs"]:
        gate_in = np.concatenate([np.array([x], np.float32), hidden], axis=1)   # [1, 8]
        z = ora.dense_forward(gate_in, w, bias, ora.IDENTITY, fused=fused)      # matmul + bias
        i = ora.activation(ora.SIGMOID, z[:, 0:4])
        u = ora.activation(ora.TANH, z[:, 4:8])
        f = ora.activation(ora.SIGMOID, z[:, 8:12])
        o = ora.activation(ora.SIGMOID, z[:, 12:16])
        cell = cell * f + i * u
        hidden = ora.activation(ora.TANH, cell) * o
        states.append(hidden.copy())
    return np.concatenate(states), cell


@pytest.mark.parametrize("fused", [True, False])
def test_lstm_fixture_pins_matmul_bias_activation(kats, fused):
    k = kats["lstm"]
    states, cell = _lstm_run(kats, fused)
    assert np.max(np.abs(states - np.array(k["lstmExpectedStates"], np.float32))) <= 1e-6
    assert np.max(np.abs(cell - np.array(k["lstmExpectedOutput"], np.float32))) <= 1e-6


def test_lstm_fixture_fails_without_bias(kats):
    # the forget-gate bias of 1 matters: dropping the bias (as operators/Matmul.swift:70 does)
    # cannot reproduce the expected states, so the fixture pins the bias term
    k = kats["lstm"]
    w = np.array(k["lstmInitialCellFusedWeights"], np.float32)
    hidden = np.array(k["lstmInitialStateHidden"], np.float32)
    cell = np.array(k["lstmInitialStateCell"], np.float32)
    x = np.array([k["lstmInputs"][0]], np.float32)
    z = ora.dense_forward(np.concatenate([x, hidden], axis=1), w, None, ora.IDENTITY)
    i, u = ora.activation(ora.SIGMOID, z[:, 0:4]), ora.activation(ora.TANH, z[:, 4:8])
    f, o = ora.activation(ora.SIGMOID, z[:, 8:12]), ora.activation(ora.SIGMOID, z[:, 12:16])
    h = ora.activation(ora.TANH, cell * f + i * u) * o
    assert np.max(np.abs(h - np.array(k["lstmExpectedStates"], np.float32)[0:1])) > 1e-3


def test_dense_activations_closed_forms():
    x = np.array([[1.0, -2.0, 0.5]], np.float32)
    w = np.array([[1.0, 0.0], [0.0, 1.0], [2.0, -2.0]], np.float32)   # x.w = [2, -3]
    b = np.array([0.5, 0.5], np.float32)                               # -> [2.5, -2.5]
    assert np.array_equal(ora.dense_forward(x, w, b, ora.RELU), [[2.5, 0.0]])
    assert np.array_equal(ora.dense_forward(x, w, b, ora.CLIPPED_RELU, coef=2.0), [[2.0, 0.0]])
    assert np.array_equal(ora.dense_forward(x, w, b, ora.IDENTITY), [[2.5, -2.5]])
    elu = ora.dense_forward(x, w, b, ora.ELU, coef=1.5)
    assert elu[0, 0] == 2.5 and abs(elu[0, 1] - 1.5 * (np.exp(-2.5) - 1)) < 1e-6
    sg = ora.dense_forward(x, w, b, ora.SIGMOID)
    assert np.allclose(sg, 1 / (1 + np.exp(-np.array([[2.5, -2.5]]))), atol=1e-6)
    # transposed weight (stored N x K) gives the same answer
    assert np.array_equal(ora.dense_forward(x, np.ascontiguousarray(w.T), b, ora.RELU, transpose_w=True), [[2.5, 0.0]])
    # bf16: fused rounds once; unfused rounds three times -- both within one bf16 ulp of the exact value
    xb, wb, bb = ora.encode(x, ora.BF16), ora.encode(w, ora.BF16), ora.encode(b, ora.BF16)
    assert np.array_equal(ora.decode(ora.dense_forward(xb, wb, bb, ora.RELU)), [[2.5, 0.0]])
    assert np.array_equal(ora.decode(ora.dense_forward(xb, wb, bb, ora.RELU, fused=False)), [[2.5, 0.0]])


# ---- element-wise neighbours and the backward of the Dense epilogue ----------------------------------
def test_elementwise_closed_forms_and_half_library_oracle():
    a = np.array([[1.5, -2.0, 0.25, 3.0]], np.float32)
    b = np.array([[0.5, 4.0, -0.25, 3.0]], np.float32)
    for dt in (ora.F32, ora.F16, ora.BF16):
        sa, sb = ora.encode(a, dt), ora.encode(b, dt)
        assert np.array_equal(ora.decode(ora.elementwise("add", sa, sb)), [[2.0, 2.0, 0.0, 6.0]])
        assert np.array_equal(ora.decode(ora.elementwise("sub", sa, sb)), [[1.0, -6.0, 0.5, 0.0]])
        assert np.array_equal(ora.decode(ora.elementwise("mul", sa, sb)), [[0.75, -8.0, -0.0625, 9.0]])
        assert np.array_equal(ora.decode(ora.elementwise("div", sa, sb)), [[3.0, -0.5, -1.0, 1.0]])
        assert np.array_equal(ora.decode(ora.elementwise("max", sa, sb)), [[1.5, 4.0, 0.25, 3.0]])
        assert np.array_equal(ora.decode(ora.elementwise("min", sa, sb)), [[0.5, -2.0, -0.25, 3.0]])
        assert np.array_equal(ora.decode(ora.elementwise("neg", sa)), -a)
    # numpy's own half arithmetic (an independent implementation) agrees with "fp32 op, round once"
    g = np.random.Generator(np.random.Philox(31))
    x = (g.standard_normal(4096) * 3).astype(np.float16)
    y = (g.standard_normal(4096) * 3).astype(np.float16)
    for op, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        assert np.array_equal(ora.elementwise(op, x, y), fn(x, y)), op
    # max is `a >= b ? a : b`: a NaN on the left gives the right operand, a NaN on the right is returned
    n = ora.elementwise("max", np.array([np.nan, 1.0], np.float32), np.array([2.0, np.nan], np.float32))
    assert n[0] == 2.0 and np.isnan(n[1])
    # broadcast of a bias row, and a scalar element
    m = ora.elementwise("add", np.ones((3, 4), np.float32), np.arange(4, dtype=np.float32))
    assert np.array_equal(m, np.ones((3, 4)) + np.arange(4))
    assert np.array_equal(ora.elementwise("mul", np.full((2, 2), 3.0, np.float32), np.array([0.5], np.float32)),
                          np.full((2, 2), 1.5))


def test_lstm_fixture_pins_the_unfused_elementwise_chain(kats):
    """The reference's LSTM states are reproduced when every step after the matmul goes through the
    oracle's element-wise functions (slices, sigmoid, tanh, mul, add) -- the chain the device runs."""
    k = kats["lstm"]
    w = np.array(k["lstmInitialCellFusedWeights"], np.float32)
    bias = np.array(k["lstmInitialCellFusedBias"], np.float32)
    cell = np.array(k["lstmInitialStateCell"], np.float32)
    hidden = np.array(k["lstmInitialStateHidden"], np.float32)
    states = []
    for x in k["lstmInputs"]:
        gate_in = np.concatenate([np.array([x], np.float32), hidden], axis=1)
        z = ora.elementwise("add", ora.matmul(gate_in, w), bias)
        i, u = ora.elementwise("sigmoid", z[:, 0:4]), ora.elementwise("tanh", z[:, 4:8])
        f, o = ora.elementwise("sigmoid", z[:, 8:12]), ora.elementwise("sigmoid", z[:, 12:16])
        cell = ora.elementwise("add", ora.elementwise("mul", cell, f), ora.elementwise("mul", i, u))
        hidden = ora.elementwise("mul", ora.elementwise("tanh", cell), o)
        states.append(hidden.copy())
    assert np.max(np.abs(np.concatenate(states) - np.array(k["lstmExpectedStates"], np.float32))) <= 1e-6
    assert np.max(np.abs(cell - np.array(k["lstmExpectedOutput"], np.float32))) <= 1e-6


def test_conversion_matches_numpy_half_and_independent_bf16():
    g = np.random.Generator(np.random.Philox(32))
    v = (g.standard_normal(8192) * 50).astype(np.float32)
    assert np.array_equal(ora.elementwise("copy", v, out_dtype=ora.F16), v.astype(np.float16))
    u = v.view(np.uint32)
    assert np.array_equal(ora.elementwise("copy", v, out_dtype=ora.BF16),
                          ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16))
    h = v.astype(np.float16)
    assert np.array_equal(ora.elementwise("copy", h, out_dtype=ora.F32), h.astype(np.float32))


def test_activation_slopes_against_numerical_derivative():
    """Pins the closed-form derivative-through-the-output used by the backward: central differences
    of the oracle's own forward activation."""
    z = np.linspace(-2.0, 2.0, 41) + 0.0123
    for kind, coef in ((ora.SIGMOID, 0.0), (ora.RELU, 0.0), (ora.TANH, 0.0), (ora.CLIPPED_RELU, 0.75),
                       (ora.ELU, 0.5), (ora.IDENTITY, 0.0)):
        def f(t):
            return np.array([ora.lib().srt_oracle_activation(kind, coef, float(v)) for v in t], np.float64)
        h = 1e-3
        numeric = (f(z + h) - f(z - h)) / (2 * h)
        got = ora.activation_slope(kind, f(z).astype(np.float32), coef)
        assert np.max(np.abs(got - numeric)) < 2e-3, kind


def test_activation_backward_bias_small_case():
    y = np.array([[0.5, -1.0], [2.0, 0.0], [1.0, 3.0]], np.float32)
    dy = np.array([[1.0, 2.0], [3.0, 4.0], [-5.0, 6.0]], np.float32)
    dx, db = ora.activation_backward_bias(y, dy, ora.RELU)
    assert np.array_equal(dx, [[1.0, 0.0], [3.0, 0.0], [-5.0, 6.0]]) and np.array_equal(db, [-1.0, 6.0])
    dx, db = ora.activation_backward_bias(y, dy, ora.IDENTITY)
    assert np.array_equal(dx, dy) and np.array_equal(db, dy.sum(axis=0))
    ys = np.array([[0.5, 0.25]], np.float32)
    dx, _ = ora.activation_backward_bias(ys, np.ones_like(ys), ora.SIGMOID)
    assert np.array_equal(dx, [[0.25, 0.1875]])
    dx, _ = ora.activation_backward_bias(ys, np.ones_like(ys), ora.TANH)
    assert np.array_equal(dx, [[0.75, 0.9375]])
