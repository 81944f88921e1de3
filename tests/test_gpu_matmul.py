"""GPU parity tests: the HIP path through the C ABI against the CPU oracle and the fp64 GEMM.

Bars: bit-exact where the arithmetic is exact (integer-valued inputs, known-answer tests);
otherwise max-norm relative error against the fp64 GEMM on the same rounded inputs
<= 1e-5 (fp32) and <= 2e-2 (bf16 / fp16), plus a tighter element-wise bound of one rounding
of the stored type.
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


@pytest.fixture(autouse=True)
def clean_plan_cache():
    """Tests that pin a plan must not leak it into the next test."""
    srt.PlanCache.clear()
    yield
    srt.PlanCache.clear()


def query_kernel(a, ta, b, tb, out):
    ad, k1 = a.descriptor()
    bd, k2 = b.descriptor()
    od, k3 = out.descriptor()
    q = srt.current_queue()
    buf = ctypes.create_string_buffer(64)
    native.check(native.lib().srtMatmulQueryKernel(ctypes.byref(ad), int(ta), ctypes.byref(bd), int(tb),
                                                   ctypes.byref(od), a.device_read(q), b.device_read(q),
                                                   out.device_read(q), buf, 64))
    return buf.value.decode()


def gpu_matmul(a_st, b_st, ta=False, tb=False, bias=None, order=srt.Order.row, want_kernel=None):
    """a_st / b_st: numpy storage arrays exactly as stored (before any transpose)."""
    a, b = srt.Tensor(a_st, order=order), srt.Tensor(b_st, order=order)
    c = srt.matmul(a, b, transposed_lhs=ta, transposed_rhs=tb,
                   bias=None if bias is None else srt.Tensor(bias))
    if want_kernel is not None:
        assert query_kernel(a, ta, b, tb, c) == want_kernel
    return c.array()


def fp64_ref(a_st, b_st, ta, tb):
    a, b = H.to64(a_st), H.to64(b_st)
    if ta:
        a = np.swapaxes(a, -1, -2)
    if tb:
        b = np.swapaxes(b, -1, -2)
    return a @ b, np.abs(a) @ np.abs(b)


def check_against_fp64(c_st, a_st, b_st, ta, tb, dt):
    c64, absprod = fp64_ref(a_st, b_st, ta, tb)
    c = H.decode(c_st)
    err = H.max_norm_rel(c, c64)
    assert err <= H.TOL[dt], f"max-norm relative error {err} exceeds {H.TOL[dt]}"
    k = a_st.shape[-2] if ta else a_st.shape[-1]
    ex = H.elementwise_excess(c, c64, absprod, dt, k)
    assert ex <= 1.0, f"element-wise error {ex} x (one rounding + fp32 accumulation bound)"
    return err


# ---- reference known-answer tests ---------------------------------------------------------------
@pytest.mark.parametrize("dt", DTS)
def test_reference_kat_2d_and_gradients(kats, dt):
    k = kats["matmul_2d"]
    a = H.encode(np.array(k["a"], np.float32), dt)
    b = H.encode(np.array(k["b"], np.float32), dt)
    ones = H.encode(np.ones((3, 4), np.float32), dt)
    assert np.array_equal(H.decode(gpu_matmul(a, b)), np.array(k["c"], np.float32))
    # matmulGradients NN case: dA = dC . B^T, dB = A^T . dC
    assert np.array_equal(H.decode(gpu_matmul(ones, b, tb=True)), np.array(k["grad_a_for_ones"], np.float32))
    assert np.array_equal(H.decode(gpu_matmul(a, ones, ta=True)), np.array(k["grad_b_for_ones"], np.float32))
    # TT
    c = np.array(k["c"], np.float32)
    assert np.array_equal(H.decode(gpu_matmul(b, a, ta=True, tb=True)), c.T)


@pytest.mark.parametrize("dt", [H.F32, H.F16])
def test_reference_kat_batched(kats, dt):
    k = kats["matmul_batched"]
    a = H.encode(np.arange(12, dtype=np.float32).reshape(2, 3, 2), dt)
    b = H.encode(np.arange(16, dtype=np.float32).reshape(2, 2, 4), dt)
    assert np.array_equal(H.decode(gpu_matmul(a, b)), np.array(k["c"], np.float32))
    ones = H.encode(np.ones((2, 3, 4), np.float32), dt)
    assert np.array_equal(H.decode(gpu_matmul(ones, b, tb=True)), np.array(k["grad_a_for_ones"], np.float32))
    assert np.array_equal(H.decode(gpu_matmul(a, ones, ta=True)), np.array(k["grad_b_for_ones"], np.float32))


def test_lstm_fixture_through_fused_dense(kats):
    """matmul + bias + sigmoid/tanh fused on the GPU reproduces the reference's LSTM states (1e-6)."""
    k = kats["lstm"]
    w = np.array(k["lstmInitialCellFusedWeights"], np.float32)
    bias = np.array(k["lstmInitialCellFusedBias"], np.float32)
    cell = np.array(k["lstmInitialStateCell"], np.float32)
    hidden = np.array(k["lstmInitialStateHidden"], np.float32)
    q = srt.current_queue()

    def gate(gate_in, lo, act):
        # one fused call per gate: column slice of W and of the bias (views, zero copy)
        wt, bt = srt.Tensor(w), srt.Tensor(bias)
        out = srt.Tensor(shape=[1, 4], dtype=np.float32)
        q.matmul(srt.Tensor(gate_in), False, wt[:, lo:lo + 4], False, out, bias=bt[lo:lo + 4], activation=act)
        return out.array()

    states = []
    for x in k["lstmInputs"]:
        gate_in = np.concatenate([np.array([x], np.float32), hidden], axis=1)
        i = gate(gate_in, 0, srt.ActivationType.sigmoid)
        u = gate(gate_in, 4, srt.ActivationType.tanh)
        f = gate(gate_in, 8, srt.ActivationType.sigmoid)
        o = gate(gate_in, 12, srt.ActivationType.sigmoid)
        cell = cell * f + i * u
        hidden = np.tanh(cell) * o
        states.append(hidden.copy())
    assert np.max(np.abs(np.concatenate(states) - np.array(k["lstmExpectedStates"], np.float32))) <= 1e-6
    assert np.max(np.abs(cell - np.array(k["lstmExpectedOutput"], np.float32))) <= 1e-6


# ---- bit-exact against the oracle on integer-valued inputs ------------------------------------------
SHAPES_ODD = [(1, 1, 1), (3, 5, 7), (17, 31, 33), (255, 257, 65), (64, 64, 64), (33, 130, 256)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_integer_inputs_bit_exact_vs_oracle(dt, ta, tb):
    r = H.rng(11)
    for (M, N, K) in SHAPES_ODD:
        kk = min(K, 64) if dt != H.F32 else K        # keep sums exactly representable in 16-bit types
        a = r.integers(-4, 5, (kk, M) if ta else (M, kk)).astype(np.float32)
        b = r.integers(-4, 5, (N, kk) if tb else (kk, N)).astype(np.float32)
        a_st, b_st = H.encode(a, dt), H.encode(b, dt)
        want = ora.matmul(a_st, b_st, ta, tb, acc=ora.ACC_F32)
        got = gpu_matmul(a_st, b_st, ta, tb)
        assert np.array_equal(got.view(np.uint16) if dt != H.F32 else got,
                              want.view(np.uint16) if dt != H.F32 else want), (M, N, K)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K,kernel", [(200, 264, 72, "mfma_64x64"), (2040, 2056, 136, "mfma_128x128"),
                                          (4000, 3976, 200, "mfma_256x256")])
def test_mfma_tiles_integer_bit_exact_and_random_vs_fp64(dt, ta, tb, M, N, K, kernel, tmp_path):
    """Aligned shapes with ragged edges in M, N and K, every tile config and staging layout."""
    # two k-contiguous operands have a 64-deep variant of the 256 x 256 kernel: cover it in their place
    if kernel == "mfma_256x256" and not ta and tb:
        kernel = "mfma_256x256_k64"
    # which of these the heuristic takes for a shape moves with its tuning: pin the tile under test
    pin_plan(tmp_path, kernel, dt, M, N, K, ta, tb)
    r = H.rng(100 + M)
    a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
    b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    got = gpu_matmul(a_st, b_st, ta, tb, want_kernel=kernel)
    exact = (np.swapaxes(a, 0, 1) if ta else a).astype(np.float64) @ (np.swapaxes(b, 0, 1) if tb else b).astype(np.float64)
    assert np.array_equal(got.view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))
    a = (r.standard_normal(a.shape) / np.sqrt(K)).astype(np.float32)
    b = r.standard_normal(b.shape).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    check_against_fp64(gpu_matmul(a_st, b_st, ta, tb), a_st, b_st, ta, tb, dt)
    srt.PlanCache.clear()


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_result_view_with_odd_pitch_takes_the_128_tile(dt):
    """A result that is a view with a row pitch that is not a multiple of 8 elements cannot take the
    256 x 256 kernels' 16-byte stores; with one 128 x 128 tile per CU or more that tile runs."""
    r = H.rng(19)
    M, N, K = 2048, 2048, 72
    a = r.integers(-3, 4, (M, K)).astype(np.float32)
    b = r.integers(-3, 4, (K, N)).astype(np.float32)
    at, bt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt))
    big = srt.Tensor(shape=[M, N + 4], dtype=at.dtype)
    out = big[:, :N]
    assert query_kernel(at, False, bt, False, out) == "mfma_128x128"
    srt.current_queue().matmul(at, False, bt, False, out)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    assert np.array_equal(out.array(), H.encode(exact.astype(np.float32), dt))
    assert np.all(H.decode(big.array()[:, N:]) == 0)          # the padding columns are untouched


@pytest.mark.parametrize("dt", DTS)
def test_random_odd_shapes_vs_oracle_and_fp64(dt):
    r = H.rng(12)
    for (M, N, K) in [(3, 5, 7), (17, 31, 33), (129, 65, 257)]:
        for ta, tb in [(False, False), (True, True)]:
            a_st = H.encode(r.uniform(-1, 1, (K, M) if ta else (M, K)), dt)
            b_st = H.encode(r.uniform(-1, 1, (N, K) if tb else (K, N)), dt)
            got = gpu_matmul(a_st, b_st, ta, tb)
            check_against_fp64(got, a_st, b_st, ta, tb, dt)
            # against the restated cpu_matmul (sequential fp32 sums): differences come from summation
            # order only, i.e. at most one unit in the last place of the stored type (plus fp32 noise)
            want = H.decode(ora.matmul(a_st, b_st, ta, tb, acc=ora.ACC_F32))
            c64, absprod = fp64_ref(a_st, b_st, ta, tb)
            tol = 2 * H.ULP[dt] * np.abs(c64) + K * 2.0 ** -22 * absprod
            assert np.all(np.abs(H.decode(got).astype(np.float64) - want) <= tol)


# ---- the benchmark configurations at full size --------------------------------------------------
def test_cfg1_f32_512_vs_oracle_and_fp64():
    r = H.rng(0)
    a = r.uniform(-1, 1, (512, 512)).astype(np.float32)
    b = r.uniform(-1, 1, (512, 512)).astype(np.float32)
    got = gpu_matmul(a, b)
    err = check_against_fp64(got, a, b, False, False, H.F32)
    want = ora.matmul(a, b)     # the reference's own arithmetic (sequential fp32)
    c64, _ = fp64_ref(a, b, False, False)
    # the GPU result is at least as close to fp64 as the reference's sequential sum is, within 2x
    assert err <= 2 * max(H.max_norm_rel(want, c64), 1e-7)


def test_f32_split_k_row_major_ragged_and_batched():
    """Row-major fp32 problems small enough for the split-K tile: ragged M, N a multiple of 4 but not
    of the tile, K a multiple of 4 but not of the 16-deep slab (and longer than one wave's prefetch),
    a batch, bias + activation.  Integer-valued inputs are bit-exact; random ones within 1e-5 of fp64."""
    r = H.rng(31)
    for (M, N, K, batch) in [(70, 132, 200, None), (33, 36, 2052, None), (96, 64, 520, 3)]:
        lead = () if batch is None else (batch,)
        a = r.integers(-3, 4, lead + (M, K)).astype(np.float32)
        b = r.integers(-3, 4, lead + (K, N)).astype(np.float32)
        got = gpu_matmul(a, b, want_kernel="f32_mfma")
        assert np.array_equal(got, (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)), (M, N, K)
        a = r.uniform(-1, 1, a.shape).astype(np.float32)
        b = r.uniform(-1, 1, b.shape).astype(np.float32)
        check_against_fp64(gpu_matmul(a, b), a, b, False, False, H.F32)
    x = r.uniform(-1, 1, (70, 200)).astype(np.float32)
    w = r.uniform(-1, 1, (200, 132)).astype(np.float32)
    bias = r.uniform(-0.5, 0.5, 132).astype(np.float32)
    y = srt.Dense(srt.Tensor(w), srt.Tensor(bias), srt.ActivationType.relu)(srt.Tensor(x)).array()
    want = np.maximum(x.astype(np.float64) @ w.astype(np.float64) + bias, 0.0)
    assert H.max_norm_rel(y, want) <= H.TOL[H.F32]


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_f32_128_tile_all_layouts_ragged(ta, tb):
    """fp32 problems large enough for the 128 x 128 tile, every transpose combination (16-byte loads
    along k or along m / n), ragged M and N edges, K that ends inside a 16-deep stage; a view with an
    unaligned pitch takes the element-wise variant of the same tile.  Bit-exact on integers, 1e-5 on
    random data, bias + relu on top."""
    r = H.rng(41)
    M, N, K = 2040, 2056, 136
    a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
    b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
    got = gpu_matmul(a, b, ta, tb, want_kernel="f32_mfma")
    exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    assert np.array_equal(got, exact.astype(np.float32))
    a = r.uniform(-1, 1, a.shape).astype(np.float32)
    b = r.uniform(-1, 1, b.shape).astype(np.float32)
    check_against_fp64(gpu_matmul(a, b, ta, tb), a, b, ta, tb, H.F32)
    bias = r.uniform(-0.5, 0.5, N).astype(np.float32)
    at, bt = srt.Tensor(a), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=np.float32)
    srt.current_queue().matmul(at, ta, bt, tb, out, bias=srt.Tensor(bias), activation=srt.ActivationType.relu)
    want = np.maximum((a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64) + bias, 0.0)
    assert H.max_norm_rel(out.array(), want) <= H.TOL[H.F32]
    if not ta and not tb:
        # operand views with a pitch that is not a multiple of 4 elements: no 16-byte loads
        av_host = r.integers(-3, 4, (M, K)).astype(np.float32)
        padded = np.zeros((M, K + 3), np.float32)
        padded[:, :K] = av_host
        av = srt.Tensor(padded)[:, :K]
        bi = r.integers(-3, 4, (K, N)).astype(np.float32)
        out2 = srt.matmul(av, srt.Tensor(bi))
        assert np.array_equal(out2.array(), (av_host.astype(np.float64) @ bi.astype(np.float64)).astype(np.float32))


def test_cfg2_f16_batched_transpose_rhs():
    r = H.rng(1)
    a = (r.standard_normal((32, 256, 256)) * 0.1).astype(np.float16)
    b = (r.standard_normal((32, 256, 256)) * 0.1).astype(np.float16)     # stored [batch, N, K]
    got = gpu_matmul(a, b, tb=True)
    check_against_fp64(got, a, b, False, True, H.F16)
    # batched == loop of single GEMMs, bit for bit
    for n in (0, 17, 31):
        assert np.array_equal(got[n].view(np.uint16), gpu_matmul(a[n], b[n], tb=True).view(np.uint16))
    # oracle restatement with fp32 accumulation on two batches (the fp16-accumulating Linux variant of the
    # reference is reported by the benchmark, not asserted: its own error is ~1e-2)
    want = ora.matmul(a[:2], b[:2], False, True, acc=ora.ACC_F32)
    assert np.max(np.abs(got[:2].astype(np.float32) - want.astype(np.float32))) <= 2.0 ** -10 * np.max(np.abs(want.astype(np.float32)))


@pytest.mark.parametrize("ta", [False, True])
def test_cfg3_bf16_8192_sampled_rows_and_invariants(ta):
    n = 8192
    r = H.rng(2)
    a = H.encode((r.standard_normal((n, n), dtype=np.float32) / np.float32(np.sqrt(n))), H.BF16)
    b = H.encode((r.standard_normal((n, n), dtype=np.float32) / np.float32(np.sqrt(n))), H.BF16)
    a_stored = np.ascontiguousarray(a.T) if ta else a
    got = gpu_matmul(a_stored, b, ta=ta, want_kernel="mfma_256x256_m16_k64")
    rows = np.unique(np.concatenate([np.arange(0, n, 131), [n - 1, 255, 256, 4095, 4096]]))
    c64 = H.to64(a[rows]) @ H.to64(b)
    absprod = np.abs(H.to64(a[rows])) @ np.abs(H.to64(b))
    c = H.decode(got[rows])
    assert H.max_norm_rel(c, c64) <= H.TOL[H.BF16]
    assert H.elementwise_excess(c, c64, absprod, H.BF16, n) <= 1.0
    cols = np.arange(5, n, 257)
    c64c = H.to64(a) @ H.to64(b[:, cols])
    assert H.max_norm_rel(H.decode(got[:, cols]), c64c) <= H.TOL[H.BF16]
    if ta:
        # same values stored transposed: same result as the untransposed call up to fp32 summation
        # order (the transposed-lhs kernel walks k from a different start per XCD), i.e. at most one
        # bf16 rounding apart
        nn = H.decode(gpu_matmul(a, b, ta=False))
        assert np.all(np.abs(H.decode(got) - nn) <= 2.0 ** -7 * np.abs(nn) + 1e-6)


def test_cfg4_dense_bf16_relu_sampled_rows():
    r = H.rng(3)
    x = H.encode(r.standard_normal((4096, 4096), dtype=np.float32), H.BF16)
    w = H.encode(r.standard_normal((4096, 11008), dtype=np.float32) / np.float32(64.0), H.BF16)
    bias = H.encode(r.uniform(-0.1, 0.1, 11008).astype(np.float32), H.BF16)
    layer = srt.Dense(srt.Tensor(w), srt.Tensor(bias), srt.ActivationType.relu)
    y = layer(srt.Tensor(x)).array()
    rows = np.arange(3, 4096, 67)
    z64 = H.to64(x[rows]) @ H.to64(w) + H.to64(bias)[None, :]
    y64 = np.maximum(z64, 0.0)
    got = H.decode(y[rows]).astype(np.float64)
    assert np.max(np.abs(got - y64)) / np.max(np.abs(y64)) <= H.TOL[H.BF16]
    assert np.all(got >= 0.0)
    absprod = np.abs(H.to64(x[rows])) @ np.abs(H.to64(w)) + 0.1
    assert np.all(np.abs(got - y64) <= 2.0 ** -8 * np.abs(y64) + 4096 * 2.0 ** -24 * absprod)
    # small slice against the oracle's fused definition: identical up to fp32 summation order
    want = H.decode(ora.dense_forward(x[:4], w[:, :256].copy(), bias[:256].copy(), ora.RELU))
    assert np.all(np.abs(H.decode(y[:4, :256]) - want) <= 2.0 ** -7 * np.abs(want) + 1e-3)


@pytest.mark.parametrize("M", [1, 8, 32])
def test_cfg5_skinny_bf16(M):
    r = H.rng(4)
    x = H.encode(r.standard_normal((M, 4096), dtype=np.float32), H.BF16)
    w = H.encode(r.standard_normal((14336, 4096), dtype=np.float32) / np.float32(64.0), H.BF16)   # stored [N, K]
    got = gpu_matmul(x, w, tb=True, want_kernel="skinny")
    check_against_fp64(got, x, w, False, True, H.BF16)
    # oracle restatement on a column slab (sequential fp32): one bf16 rounding apart at most
    want = H.decode(ora.matmul(x, w[:512], False, True, acc=ora.ACC_F32))
    assert np.all(np.abs(H.decode(got[:, :512]) - want) <= 2.0 ** -7 * np.abs(want) + 1e-3)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_skinny_ragged_and_integer_exact(dt):
    r = H.rng(40)
    for (M, N, K) in [(1, 33, 8), (5, 100, 72), (32, 1000, 520), (17, 32, 4096)]:
        x = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (N, K)).astype(np.float32)
        got = gpu_matmul(H.encode(x, dt), H.encode(w, dt), tb=True, want_kernel="skinny")
        exact = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
        assert np.array_equal(got.view(np.uint16), H.encode(exact, dt).view(np.uint16)), (M, N, K)


@pytest.mark.parametrize("tb", [True, False])
def test_skinny_fp32_integer_exact_ragged_bias_relu_batch_and_random_vs_fp64(tb, tmp_path):
    """The streaming kernel on fp32 (x . W^T and x . W, up to 32 rows): a 16-byte chunk is four k values and a 128-byte block 32 of
    them; every staged row count (8, 16, 32), K ending inside a block and of a single chunk, N not a multiple of 32, a row
    pitch wider than K, bias and relu, a batch, random operands against the fp64 product."""
    r = H.rng(41)
    q = srt.current_queue()

    def pin(M, N, K, epilogue):   # both alignment classes of the rows: the class counts eight elements whatever the type
        f = tmp_path / "plan.txt"
        lay = 21 if tb else 25
        f.write_text(f"{H.F32} {M} {N} {K} 1 {lay + 64} {epilogue} skinny\n{H.F32} {M} {N} {K} 1 {lay} {epilogue} skinny\n")
        srt.PlanCache.clear()
        srt.PlanCache.load(f)

    for (M, N, K) in [(1, 33 if tb else 36, 4), (5, 100, 72), (8, 4096, 4096), (17, 32, 4100), (32, 1000, 520), (32, 14336, 1024)]:
        x = r.integers(-3, 4, (M, K)).astype(np.float32)
        w = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        bias = r.integers(-20, 21, N).astype(np.float32)
        exact = x.astype(np.float64) @ (w.T if tb else w).astype(np.float64)
        xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(bias)
        pin(M, N, K, int(srt.ActivationType.identity) << 1)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        assert query_kernel(xt, False, wt, tb, out) == "skinny"
        q.matmul(xt, False, wt, tb, out)
        assert np.array_equal(out.array(), exact.astype(np.float32)), (M, N, K)
        pin(M, N, K, 1 | (int(srt.ActivationType.relu) << 1))
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        q.matmul(xt, False, wt, tb, out, bias=bt, activation=srt.ActivationType.relu)
        assert np.array_equal(out.array(), np.maximum(exact + bias[None, :], 0).astype(np.float32)), (M, N, K, "bias+relu")
    B_, M, N, K = 3, 20, 264, 328
    x = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (B_, N, K) if tb else (B_, K, N)).astype(np.float32)
    f = tmp_path / "plan.txt"
    f.write_text(f"{H.F32} {M} {N} {K} {B_} {85 if tb else 89} 10 skinny\n")
    srt.PlanCache.clear()
    srt.PlanCache.load(f)
    out = srt.matmul(srt.Tensor(x), srt.Tensor(w), False, tb)
    wm = np.swapaxes(w, 1, 2) if tb else w
    assert np.array_equal(out.array(), (x.astype(np.float64) @ wm.astype(np.float64)).astype(np.float32))
    M, N, K = 24, 1032, 2048
    a_st = (r.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    w_st = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    pin_plan(tmp_path, "skinny", H.F32, M, N, K, False, tb)
    check_against_fp64(gpu_matmul(a_st, w_st, False, tb, want_kernel="skinny"), a_st, w_st, False, tb, H.F32)
    srt.PlanCache.clear()


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_skinny_wide_groups_integer_exact_bias_and_batch(dt):
    """17 <= M <= 32 against a large weight: workgroups take 64 rows of W.  N not a multiple of 64 (nor of
    32), K ending inside a k block, bias + ReLU, and a strided batch that reaches the threshold together."""
    r = H.rng(41)
    for (M, N, K) in [(32, 12328, 200), (17, 12344, 72), (25, 16384, 64)]:
        x = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (N, K)).astype(np.float32)
        b = r.integers(-3, 4, N).astype(np.float32)
        xt, wt, bt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt)), srt.Tensor(H.encode(b, dt))
        out = srt.Tensor(shape=[M, N], dtype=xt.dtype)
        assert query_kernel(xt, False, wt, True, out) == "skinny"
        srt.current_queue().matmul(xt, False, wt, True, out, bias=bt, activation=srt.ActivationType.relu)
        exact = np.maximum(x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)[None, :], 0)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    B_, M, N, K = 4, 32, 3100, 136        # 4 x 49 workgroups of 64 columns
    x = r.integers(-2, 3, (B_, M, K)).astype(np.float32)
    w = r.integers(-2, 3, (B_, N, K)).astype(np.float32)
    xt, wt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt))
    out = srt.matmul(xt, wt, transposed_rhs=True)
    assert query_kernel(xt, False, wt, True, out) == "skinny"
    exact = x.astype(np.float64) @ np.swapaxes(w, 1, 2).astype(np.float64)
    assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_skinny_up_to_64_rows_integer_exact_bias_and_choice(dt, tmp_path):
    """33 <= M <= 64: two output tiles along M per workgroup, with 32 and with 64 weight rows; ragged N and K,
    bias + ReLU, a batch; and the shapes the heuristic gives to this kernel or keeps from it."""
    r = H.rng(42)
    for (M, N, K) in [(33, 1000, 520), (64, 12328, 200), (40, 12344, 72), (57, 4096, 64), (64, 264, 4096)]:
        x = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (N, K)).astype(np.float32)
        b = r.integers(-3, 4, N).astype(np.float32)
        xt, wt, bt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt)), srt.Tensor(H.encode(b, dt))
        out = srt.Tensor(shape=[M, N], dtype=xt.dtype)
        f = tmp_path / "plan.txt"
        f.write_text(f"{dt} {M} {N} {K} 1 85 10 skinny\n{dt} {M} {N} {K} 1 85 3 skinny\n")
        srt.PlanCache.clear()
        srt.PlanCache.load(f)
        assert query_kernel(xt, False, wt, True, out) == "skinny"
        srt.current_queue().matmul(xt, False, wt, True, out, bias=bt, activation=srt.ActivationType.relu)
        exact = np.maximum(x.astype(np.float64) @ w.astype(np.float64).T + b[None, :], 0)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    srt.PlanCache.clear()
    B_, M, N, K = 3, 48, 2056, 520
    x = r.integers(-2, 3, (B_, M, K)).astype(np.float32)
    w = r.integers(-2, 3, (B_, N, K)).astype(np.float32)
    xt, wt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt))
    out = srt.matmul(xt, wt, transposed_rhs=True)
    assert query_kernel(xt, False, wt, True, out) == "skinny"            # 195 workgroups of 32 rows, short k loop
    exact = x.astype(np.float64) @ np.swapaxes(w, 1, 2).astype(np.float64)
    assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_skinny_n_contiguous_weight_integer_exact_bias_and_batch(dt, tmp_path):
    """x[M, K] . W[K, N] (no transposes) with up to 64 rows of x: the streaming kernel reads W through the
    transposing LDS read.  Every staged row count, N ending inside a 64-column group, K ending inside a k block,
    bias + ReLU, a batch, and random data against fp64."""
    r = H.rng(43)
    relu = srt.ActivationType.relu
    for (M, N, K) in [(1, 64, 8), (5, 104, 72), (8, 1000, 520), (16, 4096, 64), (17, 12328, 200), (32, 264, 4096),
                      (33, 1000, 520), (64, 12344, 72), (57, 4096, 192)]:
        x = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (K, N)).astype(np.float32)
        b = r.integers(-3, 4, N).astype(np.float32)
        xt, wt, bt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt)), srt.Tensor(H.encode(b, dt))
        out = srt.Tensor(shape=[M, N], dtype=xt.dtype)
        pin_plan(tmp_path, "skinny", dt, M, N, K, False, False)
        assert query_kernel(xt, False, wt, False, out) == "skinny"
        srt.current_queue().matmul(xt, False, wt, False, out)
        exact = x.astype(np.float64) @ w.astype(np.float64)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
        pin_plan(tmp_path, "skinny", dt, M, N, K, False, False, bias=True, act=relu)
        srt.current_queue().matmul(xt, False, wt, False, out, bias=bt, activation=relu)
        exact = np.maximum(exact + b[None, :], 0)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    B_, M, N, K = 3, 24, 2056, 136
    x = r.integers(-2, 3, (B_, M, K)).astype(np.float32)
    w = r.integers(-2, 3, (B_, K, N)).astype(np.float32)
    f = tmp_path / "plan.txt"
    f.write_text(f"{dt} {M} {N} {K} {B_} 89 0 skinny\n")
    srt.PlanCache.clear()
    srt.PlanCache.load(f)
    xt, wt = srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt))
    out = srt.matmul(xt, wt)
    assert query_kernel(xt, False, wt, False, out) == "skinny"
    exact = x.astype(np.float64) @ w.astype(np.float64)
    assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))
    M, N, K = 48, 2048, 4096
    pin_plan(tmp_path, "skinny", dt, M, N, K, False, False)
    a = (r.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    w = r.standard_normal((K, N)).astype(np.float32)
    a_st, w_st = H.encode(a, dt), H.encode(w, dt)
    check_against_fp64(gpu_matmul(a_st, w_st, want_kernel="skinny"), a_st, w_st, False, False, dt)
    srt.PlanCache.clear()


# ---- layouts: views, column-major, strided output ------------------------------------------------------
@pytest.mark.parametrize("dt", DTS)
def test_strided_views_and_column_major(dt):
    r = H.rng(13)
    big_a = H.encode(r.integers(-4, 5, (40, 48)).astype(np.float32), dt)
    big_b = H.encode(r.integers(-4, 5, (48, 56)).astype(np.float32), dt)
    ta, tb = srt.Tensor(big_a), srt.Tensor(big_b)
    va, vb = ta[1:33:2, 2:47:3], tb[3:18, 1:53:4]          # both strides non-unit, offset base pointers
    got = srt.matmul(va, vb).array()
    want = ora.matmul(big_a[1:33:2, 2:47:3], big_b[3:18, 1:53:4], acc=ora.ACC_F32)
    assert np.array_equal(got.view(np.uint16) if dt != H.F32 else got, want.view(np.uint16) if dt != H.F32 else want)
    # column-major operands and result (result order follows lhs.order)
    ca, cb = srt.Tensor(big_a, order=srt.Order.col), srt.Tensor(big_b, order=srt.Order.col)
    cc = srt.matmul(ca, cb)
    assert cc.order == srt.Order.col and cc.strides == (1, 40)
    want = ora.matmul(big_a, big_b, acc=ora.ACC_F32)
    assert np.array_equal(H.decode(cc.array()), H.decode(want))
    # .t views as operands equal the transposed: flags
    assert np.array_equal(H.decode(srt.matmul(ta.t, tb.t, transposed_lhs=True, transposed_rhs=True).array()), H.decode(want))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_unaligned_operands_run_on_the_matrix_cores(dt):
    """Operands the 16-byte loaders cannot take -- odd extents and row pitches, views with both strides non-unit
    or an odd start, a strided result -- go through element-wise staging into the same MFMA tiles: bit-exact on
    integers for every transpose combination, both tile sizes, bias + ReLU, a batch; fp64 bound on random data."""
    r = H.rng(130)
    relu = srt.ActivationType.relu
    for (M, N, K, ta, tb) in [(33, 33, 33, False, False), (129, 67, 100, True, False), (70, 131, 65, False, True),
                              (65, 65, 129, True, True), (2049, 2051, 77, False, False), (2050, 2049, 70, True, True)]:
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        bias = r.integers(-3, 4, N).astype(np.float32)
        at, bt, biast = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt)), srt.Tensor(H.encode(bias, dt))
        out = srt.Tensor(shape=[M, N], dtype=at.dtype)
        assert query_kernel(at, ta, bt, tb, out) == ("mfma_128x128_any" if M > 2000 else "mfma_64x64_any")
        srt.current_queue().matmul(at, ta, bt, tb, out, bias=biast, activation=relu)
        exact = np.maximum((a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64) + bias[None, :], 0)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K, ta, tb)
    # views: both strides non-unit, odd starts; then a batch of odd-pitch matrices
    big_a = r.integers(-3, 4, (300, 200)).astype(np.float32)
    big_b = r.integers(-3, 4, (200, 400)).astype(np.float32)
    ta_, tb_ = srt.Tensor(H.encode(big_a, dt)), srt.Tensor(H.encode(big_b, dt))
    va, vb = ta_[1:291:2, 3:198:3], tb_[5:70, 1:391:3]
    got = srt.matmul(va, vb)
    assert query_kernel(va, False, vb, False, got) == "mfma_64x64_any"
    exact = big_a[1:291:2, 3:198:3].astype(np.float64) @ big_b[5:70, 1:391:3].astype(np.float64)
    assert np.array_equal(got.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))
    x = r.integers(-3, 4, (3, 70, 45)).astype(np.float32)
    w = r.integers(-3, 4, (3, 45, 99)).astype(np.float32)
    got = srt.matmul(srt.Tensor(H.encode(x, dt)), srt.Tensor(H.encode(w, dt)))
    assert np.array_equal(got.array().view(np.uint16), H.encode((x.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), dt).view(np.uint16))
    # random data against fp64
    M, N, K = 515, 1001, 777
    a = (r.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    check_against_fp64(gpu_matmul(a_st, b_st, want_kernel="mfma_64x64_any"), a_st, b_st, False, False, dt)


def test_column_major_bias_broadcast_direction():
    r = H.rng(14)
    x = r.integers(-3, 4, (24, 16)).astype(np.float32)
    w = r.integers(-3, 4, (16, 40)).astype(np.float32)
    b = r.integers(-3, 4, 40).astype(np.float32)
    xt, wt = srt.Tensor(x, order=srt.Order.col), srt.Tensor(w, order=srt.Order.col)
    out = srt.matmul(xt, wt, bias=srt.Tensor(b))
    assert np.array_equal(out.array(), x @ w + b[None, :])


@pytest.mark.parametrize("act", list(srt.ActivationType))
@pytest.mark.parametrize("dt", DTS)
def test_every_activation_vs_oracle(act, dt):
    r = H.rng(15)
    x = H.encode(r.standard_normal((72, 64)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((64, 136)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, 136).astype(np.float32), dt)
    coef = 0.75
    layer = srt.Dense(srt.Tensor(w), srt.Tensor(b), act, relu_ceiling=coef, elu_alpha=coef)
    got = H.decode(layer(srt.Tensor(x)).array())
    want = H.decode(ora.dense_forward(x, w, b, int(act), coef=coef, acc=ora.ACC_F32, fused=True))
    tol = {H.F32: 2e-6, H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("act", list(srt.ActivationType))
def test_ring_kernel_epilogues_vs_oracle(act, dt, tmp_path):
    """Every activation (+ bias) through the 256 x 256 ring kernel, ragged M / N / K edges."""
    r = H.rng(16)
    M, N, K = 3600, 3592, 72
    pin_plan_for_shape(tmp_path, "mfma_256x256", dt, M, N, K)
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    xt, wt = srt.Tensor(x), srt.Tensor(w)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    assert query_kernel(xt, False, wt, False, out) == "mfma_256x256"
    layer = srt.Dense(wt, srt.Tensor(b), act, relu_ceiling=coef, elu_alpha=coef)
    got = H.decode(layer(xt).array())
    rows = np.concatenate([np.arange(0, M, 211), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, acc=ora.ACC_F32, fused=True))
    tol = {H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got[rows] - want) <= tol * np.maximum(np.abs(want), 1.0))


# ---- the 256 x 256 ring kernel on 16x16x32 MFMAs ----------------------------------------------------
def pin_m16(tmp_path, dt, M, N, K, ta, tb, batch=1, bias=False, act=srt.ActivationType.identity):
    """The heuristic takes this kernel for a full device and a long k loop only: pin it for a small shape."""
    layout = (2 if ta else 1) | (4 if tb else 8) | 16 | 64
    epilogue = (1 if bias else 0) | (int(act) << 1)
    f = tmp_path / "plan.txt"
    f.write_text(f"{dt} {M} {N} {K} {batch} {layout} {epilogue} mfma_256x256_m16\n")
    srt.PlanCache.clear()
    srt.PlanCache.load(f)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_m16_kernel_integer_bit_exact_and_random_vs_fp64(dt, ta, tb, tmp_path):
    """Every staging layout; ragged edges in M and N, K of one stage, ending inside a stage, with an
    even and an odd number of stages, fewer stages than the ring holds; several tiles per workgroup."""
    r = H.rng(300)
    for (M, N, K) in [(512, 512, 32), (512, 768, 160), (1000, 520, 72), (2048, 2056, 200), (4400, 4360, 328)]:
        pin_m16(tmp_path, dt, M, N, K, ta, tb)
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        got = gpu_matmul(H.encode(a, dt), H.encode(b, dt), ta, tb, want_kernel="mfma_256x256_m16")
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(got.view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    M, N, K = 2040, 2056, 264
    pin_m16(tmp_path, dt, M, N, K, ta, tb)
    a = (r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32)
    b = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    check_against_fp64(gpu_matmul(a_st, b_st, ta, tb, want_kernel="mfma_256x256_m16"), a_st, b_st, ta, tb, dt)
    srt.PlanCache.clear()


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("act", list(srt.ActivationType))
@pytest.mark.parametrize("tw", [False, True])
def test_m16_kernel_epilogues_vs_oracle(act, dt, tw, tmp_path):
    """y = act(x . W + b) and act(x . W^T + b): every activation through the fused epilogue, ragged M / N
    edges and a K that ends inside a stage."""
    r = H.rng(19)
    M, N, K = 2100, 2056, 200
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((N, K) if tw else (K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    pin_m16(tmp_path, dt, M, N, K, False, tw, bias=True, act=act)
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    srt.current_queue().matmul(xt, False, wt, tw, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 131), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=tw,
                                      acc=ora.ACC_F32, fused=True))
    tol = {H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got[rows] - want) <= tol * np.maximum(np.abs(want), 1.0))
    srt.PlanCache.clear()


def test_m16_kernel_batched_short_k_and_nan(tmp_path):
    """Strided batch, K shorter than one stage (8) and of one, two and three stages, a NaN row."""
    r = H.rng(20)
    for K in (8, 32, 72, 136, 192):
        B_, M, N = 3, 1024, 1032
        a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
        w = r.integers(-3, 4, (B_, K, N)).astype(np.float32)
        pin_m16(tmp_path, H.BF16, M, N, K, False, False, batch=B_)
        at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
        out = srt.matmul(at, wt)
        assert query_kernel(at, False, wt, False, out) == "mfma_256x256_m16"
        exact = a.astype(np.float64) @ w.astype(np.float64)
        assert np.array_equal(out.array(), H.encode(exact.astype(np.float32), H.BF16)), K
    M = N = 1536
    a = np.zeros((M, 64), np.float32)
    w = np.zeros((64, N), np.float32)
    a[:, 0] = 1.0
    w[0, :] = 2.0
    a[5, 1] = np.nan
    w[1, :] = 1.0
    pin_m16(tmp_path, H.BF16, M, N, 64, False, False)
    got = gpu_matmul(H.encode(a, H.BF16), H.encode(w, H.BF16), want_kernel="mfma_256x256_m16")
    assert np.all(got[5] == 0x7FFF) and np.all(got[6] == H.encode(np.array([2.0], np.float32), H.BF16)[0])
    srt.PlanCache.clear()


# ---- split-K over the 256 x 256 kernel --------------------------------------------------------------
def pin_plan_for_shape(tmp_path, plan, dt, M, N, K, batch=1):
    """Pins `plan` for a shape under every layout class and epilogue (and for the transposed problem a
    column-major call turns into), for tests of one kernel that should not move with the heuristic."""
    f = tmp_path / "plan_shape.txt"
    f.write_text("".join(f"{dt} {m} {n} {K} {batch} {layout} {epi} {plan}\n"
                         for (m, n) in ((M, N), (N, M)) for layout in range(128) for epi in range(14)))
    srt.PlanCache.clear()
    srt.PlanCache.load(f)


def pin_plan(tmp_path, plan, dt, M, N, K, ta, tb, bias=False, act=srt.ActivationType.identity):
    layout = (2 if ta else 1) | (4 if tb else 8) | 16 | 64
    f = tmp_path / "plan.txt"
    f.write_text(f"{dt} {M} {N} {K} 1 {layout} {(1 if bias else 0) | (int(act) << 1)} {plan}\n")
    srt.PlanCache.clear()
    srt.PlanCache.load(f)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_splitk_integer_bit_exact_and_random_vs_fp64(dt, ta, tb, tmp_path):
    """K cut into 2, 4 and 8 parts; ragged M and N edges; every staging layout."""
    r = H.rng(310)
    for (M, N, K) in [(512, 520, 1024), (304, 264, 2048), (200, 1032, 4096), (96, 520, 2048), (128, 264, 4096)]:
        pin_plan(tmp_path, "mfma_256x256_splitk", dt, M, N, K, ta, tb)
        a = r.integers(-2, 3, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-2, 3, (N, K) if tb else (K, N)).astype(np.float32)
        got = gpu_matmul(H.encode(a, dt), H.encode(b, dt), ta, tb, want_kernel="mfma_256x256_splitk")
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(got.view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    M, N, K = 520, 776, 2048
    pin_plan(tmp_path, "mfma_256x256_splitk", dt, M, N, K, ta, tb)
    a = (r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32)
    b = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    check_against_fp64(gpu_matmul(a_st, b_st, ta, tb, want_kernel="mfma_256x256_splitk"), a_st, b_st, ta, tb, dt)
    srt.PlanCache.clear()


@pytest.mark.parametrize("act", list(srt.ActivationType))
def test_splitk_epilogues_vs_oracle_and_nan(act, tmp_path):
    """Bias and every activation are applied once, after the parts are added; a NaN survives."""
    r = H.rng(311)
    dt = H.BF16
    M, N, K = 520, 264, 2048
    x = H.encode(r.standard_normal((M, K)).astype(np.float32) / 8, dt)
    w = H.encode((r.standard_normal((K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    pin_plan(tmp_path, "mfma_256x256_splitk", dt, M, N, K, False, False, bias=True, act=act)
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    srt.current_queue().matmul(xt, False, wt, False, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 37), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=False,
                                      acc=ora.ACC_F32, fused=True))
    assert np.all(np.abs(got[rows] - want) <= 2.0 ** -7 * np.maximum(np.abs(want), 1.0))
    if act == srt.ActivationType.identity:
        a = np.zeros((M, K), np.float32)
        a[:, 0] = 1.0
        a[5, K - 1] = np.nan                      # lands in the last part only
        pin_plan(tmp_path, "mfma_256x256_splitk", dt, M, N, K, False, False)
        got = gpu_matmul(H.encode(a, dt), w, want_kernel="mfma_256x256_splitk")
        assert np.all(got[5] == 0x7FFF) and not np.any(got[6] == 0x7FFF)
    srt.PlanCache.clear()


def test_splitk_is_the_choice_for_few_tiles_and_long_k():
    a = srt.Tensor(H.encode(np.zeros((128, 4096), np.float32), H.BF16))
    b = srt.Tensor(H.encode(np.zeros((4096, 2048), np.float32), H.BF16))
    out = srt.Tensor(shape=[128, 2048], dtype=a.dtype)
    assert query_kernel(a, False, b, False, out) == "mfma_256x256_splitk"      # eight half tiles in eight parts
    a2 = srt.Tensor(H.encode(np.zeros((128, 2048), np.float32), H.BF16))       # K = 2048: not worth the extra pass
    b2 = srt.Tensor(H.encode(np.zeros((2048, 2048), np.float32), H.BF16))
    assert query_kernel(a2, False, b2, False, out) != "mfma_256x256_splitk"
    a3 = srt.Tensor(H.encode(np.zeros((512, 4096), np.float32), H.BF16))       # 128 quarter tiles: one round of those instead
    b3 = srt.Tensor(H.encode(np.zeros((4096, 4096), np.float32), H.BF16))
    out3 = srt.Tensor(shape=[512, 4096], dtype=a.dtype)
    assert query_kernel(a3, False, b3, False, out3) == "mfma_128x128_m16_k128"


# ---- fp32: the k range in parts over the 128 x 128 tiles ------------------------------------------------
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_f32_tile_parts_integer_bit_exact_bias_relu_and_random_vs_fp64(ta, tb, tmp_path):
    """fp32 problems of fewer 128 x 128 tiles than two per compute unit run their k range in 2-16 parts with the sums in
    a second kernel: integer operands bit-exact (parts of 256, 512 and 1024 k; ragged M and N; N not a multiple of 4 with a
    k-contiguous B; bias and relu applied after the sum), then random operands against the fp64 product -- pinned and as
    the heuristic's own choice."""
    r = H.rng(330)
    PARTS = "f32_mfma_128x128_parts"
    shapes = [(512, 1024, 1024), (520, 1000, 2048), (136, 264, 4096), (2048, 2048, 512)]
    if tb:
        shapes.append((200, 1001, 1024))
    for (M, N, K) in shapes:
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        bias = r.integers(-20, 21, N).astype(np.float32)
        at, bt, biast = srt.Tensor(a), srt.Tensor(b), srt.Tensor(bias)
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        for pinned in (True, False):
            srt.PlanCache.clear()
            if pinned:
                pin_plan(tmp_path, PARTS, H.F32, M, N, K, ta, tb)
            out = srt.Tensor(shape=[M, N], dtype=np.float32)
            assert query_kernel(at, ta, bt, tb, out) == "f32_mfma"
            srt.current_queue().matmul(at, ta, bt, tb, out)
            assert np.array_equal(out.array(), exact.astype(np.float32)), (M, N, K, pinned)
        srt.PlanCache.clear()
        pin_plan(tmp_path, PARTS, H.F32, M, N, K, ta, tb, bias=True, act=srt.ActivationType.relu)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(at, ta, bt, tb, out, bias=biast, activation=srt.ActivationType.relu)
        assert np.array_equal(out.array(), np.maximum(exact + bias[None, :], 0).astype(np.float32)), (M, N, K, "bias+relu")
    M, N, K = 1000, 1032, 2048
    a_st = (r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32)
    b_st = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    pin_plan(tmp_path, PARTS, H.F32, M, N, K, ta, tb)
    check_against_fp64(gpu_matmul(a_st, b_st, ta, tb, want_kernel="f32_mfma"), a_st, b_st, ta, tb, H.F32)
    srt.PlanCache.clear()


# ---- fp32: the ring kernel in its three tile shapes ----------------------------------------------------------
@pytest.mark.parametrize("RING", ["f32_mfma_128x128_ring", "f32_mfma_64x128_ring", "f32_mfma_64x64_ring"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_f32_ring_kernel_integer_bit_exact_bias_relu_batch_and_random_vs_fp64(ta, tb, RING, tmp_path):
    """Every staging layout and tile shape of the fp32 ring kernel; k loops of two, three and an odd number of 64-deep
    units; ragged edges in M and N (a last tile of 8 rows, of 4 columns); one tile and several per workgroup (1225 tiles
    of 128 x 128); fewer tiles than workgroups; bias and relu; a strided batch; then random operands against the fp64
    product."""
    r = H.rng(340)
    for (M, N, K) in [(256, 384, 128), (1000, 516, 192), (2048, 2056, 320), (4400, 4356, 128), (136, 132, 1152)]:
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        bias = r.integers(-20, 21, N).astype(np.float32)
        at, bt, biast = srt.Tensor(a), srt.Tensor(b), srt.Tensor(bias)
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(at, ta, bt, tb, out)
        assert np.array_equal(out.array(), exact.astype(np.float32)), (M, N, K)
        pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb, bias=True, act=srt.ActivationType.relu)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(at, ta, bt, tb, out, bias=biast, activation=srt.ActivationType.relu)
        assert np.array_equal(out.array(), np.maximum(exact + bias[None, :], 0).astype(np.float32)), (M, N, K, "bias+relu")
        if K > 192:
            continue
        # the other forms of the store code: a bias alone, relu alone, an activation switched per element
        pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb, bias=True)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(at, ta, bt, tb, out, bias=biast)
        assert np.array_equal(out.array(), (exact + bias[None, :]).astype(np.float32)), (M, N, K, "bias")
        pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb, act=srt.ActivationType.relu)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(at, ta, bt, tb, out, activation=srt.ActivationType.relu)
        assert np.array_equal(out.array(), np.maximum(exact, 0).astype(np.float32)), (M, N, K, "relu")
        pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb, bias=True, act=srt.ActivationType.tanh)
        out = srt.Tensor(shape=[M, N], dtype=np.float32)
        srt.current_queue().matmul(srt.Tensor(a / 64), ta, bt, tb, out, bias=srt.Tensor(bias / 16), activation=srt.ActivationType.tanh)
        want = np.tanh(exact / 64 + bias[None, :].astype(np.float64) / 16)   # the products and sums stay exact at this scale
        assert np.max(np.abs(out.array() - want)) <= 1e-6, (M, N, K, "bias+tanh")
    B_, M, N, K = 3, 520, 392, 256
    a = r.integers(-3, 4, (B_, K, M) if ta else (B_, M, K)).astype(np.float32)
    b = r.integers(-3, 4, (B_, N, K) if tb else (B_, K, N)).astype(np.float32)
    f = tmp_path / "plan.txt"
    layout = (2 if ta else 1) | (4 if tb else 8) | 16 | 64
    f.write_text(f"{H.F32} {M} {N} {K} {B_} {layout} {int(srt.ActivationType.identity) << 1} {RING}\n")
    srt.PlanCache.clear()
    srt.PlanCache.load(f)
    out = srt.matmul(srt.Tensor(a), srt.Tensor(b), ta, tb)
    am = np.swapaxes(a, 1, 2) if ta else a
    bm = np.swapaxes(b, 1, 2) if tb else b
    assert np.array_equal(out.array(), (am.astype(np.float64) @ bm.astype(np.float64)).astype(np.float32))
    M, N, K = 1000, 1032, 2048
    a_st = (r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32)
    b_st = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    pin_plan(tmp_path, RING, H.F32, M, N, K, ta, tb)
    check_against_fp64(gpu_matmul(a_st, b_st, ta, tb, want_kernel="f32_mfma"), a_st, b_st, ta, tb, H.F32)
    srt.PlanCache.clear()


# ---- the 128 x 256 form of the 16x16x32 kernel ---------------------------------------------------------
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("tb", [False, True])
def test_m16_half_tile_integer_bit_exact_random_and_batched(dt, tb, tmp_path):
    """k-contiguous A against both B layouts; ragged edges in M (not a multiple of 128) and N, K below one
    stage, ending inside a stage, fewer stages than the ring holds; several tiles per workgroup; a batch."""
    r = H.rng(320)
    for (M, N, K) in [(128, 256, 32), (136, 264, 8), (1000, 776, 200), (2048, 2056, 328), (4360, 4360, 72)]:
        pin_plan(tmp_path, "mfma_128x256_m16", dt, M, N, K, False, tb)
        a = r.integers(-3, 4, (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        got = gpu_matmul(H.encode(a, dt), H.encode(b, dt), False, tb, want_kernel="mfma_128x256_m16")
        exact = a.astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(got.view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    M, N, K = 1160, 1032, 264
    pin_plan(tmp_path, "mfma_128x256_m16", dt, M, N, K, False, tb)
    a = (r.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    b = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    a_st, b_st = H.encode(a, dt), H.encode(b, dt)
    check_against_fp64(gpu_matmul(a_st, b_st, False, tb, want_kernel="mfma_128x256_m16"), a_st, b_st, False, tb, dt)
    srt.PlanCache.clear()
    # the heuristic's own choice, batched: 3 x 6 x 4 half tiles
    B_, M, N, K = 3, 768, 1024, 520
    a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (B_, N, K) if tb else (B_, K, N)).astype(np.float32)
    at, wt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(w, dt))
    out = srt.matmul(at, wt, transposed_rhs=tb)
    if not tb:
        assert query_kernel(at, False, wt, tb, out) == "mfma_128x256_m16"
    exact = a.astype(np.float64) @ (np.swapaxes(w, 1, 2) if tb else w).astype(np.float64)
    assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16))


@pytest.mark.parametrize("act", list(srt.ActivationType))
def test_m16_half_tile_epilogues_vs_oracle_and_nan(act, tmp_path):
    r = H.rng(321)
    dt = H.BF16
    M, N, K = 1100, 520, 200
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    pin_plan(tmp_path, "mfma_128x256_m16", dt, M, N, K, False, False, bias=True, act=act)
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    srt.current_queue().matmul(xt, False, wt, False, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 61), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=False,
                                      acc=ora.ACC_F32, fused=True))
    assert np.all(np.abs(got[rows] - want) <= 2.0 ** -7 * np.maximum(np.abs(want), 1.0))
    if act == srt.ActivationType.identity:
        a = np.zeros((M, 64), np.float32)
        w2 = np.zeros((64, N), np.float32)
        a[:, 0] = 1.0
        w2[0, :] = 2.0
        a[5, 1] = np.nan
        w2[1, :] = 1.0
        pin_plan(tmp_path, "mfma_128x256_m16", dt, M, N, 64, False, False)
        got = gpu_matmul(H.encode(a, dt), H.encode(w2, dt), want_kernel="mfma_128x256_m16")
        assert np.all(got[5] == 0x7FFF) and np.all(got[6] == H.encode(np.array([2.0], np.float32), dt)[0])
    srt.PlanCache.clear()


def test_m16_kernels_are_the_choice_for_a_full_device():
    """From half a device up: the 64-deep form when K is a whole number of 64-deep units (at least eight), else
    the 32-deep one."""
    a = srt.Tensor(H.encode(np.zeros((4096, 2048), np.float32), H.BF16))
    b = srt.Tensor(H.encode(np.zeros((2048, 4096), np.float32), H.BF16))
    out = srt.Tensor(shape=[4096, 4096], dtype=a.dtype)
    assert query_kernel(a, False, b, False, out) == "mfma_256x256_m16_k64"
    assert query_kernel(a, False, srt.Tensor(H.encode(np.zeros((4096, 2048), np.float32), H.BF16)), True, out) == \
        "mfma_256x256_m16_k64"
    a2 = srt.Tensor(H.encode(np.zeros((4096, 2080), np.float32), H.BF16))      # K = 2080 = 32.5 units
    b2 = srt.Tensor(H.encode(np.zeros((2080, 4096), np.float32), H.BF16))
    assert query_kernel(a2, False, b2, False, out) == "mfma_256x256_m16"


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("act", list(srt.ActivationType))
def test_k64_kernel_epilogues_vs_oracle(act, dt):
    """y = act(x . W^T + b) with W stored [N, K] (both operands k-contiguous): every activation through
    the 64-deep 256 x 256 kernel; ragged M / N edges and a K that ends inside a stage."""
    r = H.rng(17)
    M, N, K = 3600, 3592, 200
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((N, K)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    assert query_kernel(xt, False, wt, True, out) == "mfma_256x256_k64"
    srt.current_queue().matmul(xt, False, wt, True, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 211), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=True,
                                      acc=ora.ACC_F32, fused=True))
    tol = {H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got[rows] - want) <= tol * np.maximum(np.abs(want), 1.0))


def test_k64_kernel_batched_short_k_and_nan(tmp_path):
    """Strided batch, K shorter than one stage (8) and of one, two and three stages, a NaN row."""
    r = H.rng(18)
    for K in (8, 64, 72, 136, 192):
        B_, M, N = 3, 2048, 2056
        a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
        w = r.integers(-3, 4, (B_, N, K)).astype(np.float32)
        at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
        pin_plan_for_shape(tmp_path, "mfma_256x256_k64", H.BF16, M, N, K, batch=B_)
        out = srt.matmul(at, wt, transposed_rhs=True)
        assert query_kernel(at, False, wt, True, out) == "mfma_256x256_k64"
        exact = a.astype(np.float64) @ np.swapaxes(w, 1, 2).astype(np.float64)
        assert np.array_equal(out.array(), H.encode(exact.astype(np.float32), H.BF16)), K
    a = np.zeros((3584, 64), np.float32)
    w = np.zeros((3584, 64), np.float32)
    a[:, 0] = 1.0
    w[:, 0] = 2.0
    a[5, 1] = np.nan
    w[:, 1] = 1.0
    pin_plan_for_shape(tmp_path, "mfma_256x256_k64", H.BF16, 3584, 3584, 64)
    got = gpu_matmul(H.encode(a, H.BF16), H.encode(w, H.BF16), tb=True, want_kernel="mfma_256x256_k64")
    assert np.all(got[5] == 0x7FFF) and np.all(got[6] == H.encode(np.array([2.0], np.float32), H.BF16)[0])


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_ring_kernel_batched_broadcast_and_column_major(dt, tmp_path):
    """Rank-3 operands through the 256 x 256 ring kernel: strided batch, a broadcast (stride 0) weight,
    and a column-major problem (computed as C^T, bias then broadcast along the other dimension)."""
    r = H.rng(17)
    B_, M, N, K = 3, 2048, 2304, 40
    a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (K, N)).astype(np.float32)
    a_st, w_st = H.encode(a, dt), H.encode(w, dt)
    at = srt.Tensor(a_st)
    w3 = srt.Tensor(np.broadcast_to(w_st, (B_, K, N)).copy())
    out = srt.Tensor(shape=[B_, M, N], dtype=a_st.dtype)
    pin_plan_for_shape(tmp_path, "mfma_256x256", dt, M, N, K, batch=B_)
    assert query_kernel(at, False, w3, False, out) == "mfma_256x256"
    got = srt.matmul(at, w3).array()
    exact = H.encode((a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), dt)
    assert np.array_equal(got.view(np.uint16), exact.view(np.uint16))
    # broadcast weight: same storage for every batch (batch stride 0), built as a view descriptor by hand
    q = srt.current_queue()
    wt = srt.Tensor(w_st)
    ad, k1 = at.descriptor()
    bd, k2 = native.make_descriptor(native.REAL16F if dt == H.F16 else native.REAL16BF, (B_, K, N), (0, N, 1), native.ORDER_ROW)
    od, k3 = out.descriptor()
    native.check(native.lib().srtMatmul(at.device_read(q), ctypes.byref(ad), 0, wt.device_read(q), ctypes.byref(bd), 0,
                                        out.device_read_write(q), ctypes.byref(od), q.stream))
    assert np.array_equal(out.array().view(np.uint16), exact.view(np.uint16))
    # column-major 2-D problem with bias: result order follows lhs.order; bias still runs along N
    M2, N2, K2 = 3584, 3840, 48
    x = r.integers(-3, 4, (M2, K2)).astype(np.float32)
    w2 = r.integers(-3, 4, (K2, N2)).astype(np.float32)
    b2 = r.integers(-3, 4, N2).astype(np.float32)
    xc, wc = srt.Tensor(H.encode(x, dt), order=srt.Order.col), srt.Tensor(H.encode(w2, dt), order=srt.Order.col)
    pin_plan_for_shape(tmp_path, "mfma_256x256", dt, M2, N2, K2)
    yc = srt.matmul(xc, wc, bias=srt.Tensor(H.encode(b2, dt)))
    assert yc.order == srt.Order.col and query_kernel(xc, False, wc, False, yc) == "mfma_256x256"
    want = H.encode((x.astype(np.float64) @ w2.astype(np.float64) + b2.astype(np.float64)[None, :]).astype(np.float32), dt)
    assert np.array_equal(yc.array().view(np.uint16), want.view(np.uint16))
    # and relu on top (bias per row after the transposition inside the library)
    layer = srt.Dense(wc, srt.Tensor(H.encode(b2, dt)), srt.ActivationType.relu)
    assert np.array_equal(layer(xc).array().view(np.uint16), H.encode(np.maximum(H.decode(want), 0), dt).view(np.uint16))
    srt.PlanCache.clear()


def test_ring_kernel_nan_and_inf_encode_like_the_reference(tmp_path):
    """A NaN anywhere in a tile switches the wave to the exact encoder: NaN -> 0x7FFF, inf stays inf."""
    M = N = 3584
    K = 64
    pin_plan_for_shape(tmp_path, "mfma_256x256", H.BF16, M, N, K)
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    a[:, 0] = 1.0
    b[0, :] = 2.0
    a[5, 1] = np.nan       # row 5 of C becomes NaN
    a[300, 2] = np.inf     # row 300 becomes inf (inf * 0 products avoided: only column k=2 of b is nonzero below)
    b[2, :] = 1.0
    b[1, :] = 1.0
    got = gpu_matmul(H.encode(a, H.BF16), H.encode(b, H.BF16), want_kernel="mfma_256x256")
    assert np.all(got[5] == 0x7FFF)
    assert np.all(got[300] == 0x7F80)
    assert np.all(got[6] == H.encode(np.array([2.0], np.float32), H.BF16)[0])
    # relu maps the NaN row to 0 (x > 0 ? x : 0), identity keeps it
    layer = srt.Dense(srt.Tensor(H.encode(b, H.BF16)), None, srt.ActivationType.relu)
    y = layer(srt.Tensor(H.encode(a, H.BF16))).array()
    assert np.all(y[5] == 0) and np.all(y[300] == 0x7F80)
    srt.PlanCache.clear()


# ---- error behaviour -----------------------------------------------------------------------------
def test_not_supported_and_invalid_value_surface_as_in_the_reference():
    q = srt.current_queue()
    a = srt.Tensor(np.zeros((4, 4), np.float32))
    out = srt.Tensor(shape=[4, 4], dtype=np.float32)
    ad, k1 = native.make_descriptor(native.REAL64F, (4, 4), (4, 1), native.ORDER_ROW)
    st = native.lib().srtMatmul(a.device_read(q), ctypes.byref(ad), 0, a.device_read(q), ctypes.byref(ad), 0,
                                out.device_read_write(q), ctypes.byref(ad), q.stream)
    assert st == native.ERROR_NOT_SUPPORTED          # caller runs its CPU fallback
    with pytest.raises(srt.NotSupportedError):
        native.check(st)
    with pytest.raises(ValueError):
        srt.matmul(a, srt.Tensor(np.zeros((3, 4), np.float32)))


def test_empty_extents_launch_nothing():
    a = srt.Tensor(shape=[0, 8], dtype=np.float32)
    b = srt.Tensor(np.zeros((8, 4), np.float32))
    assert srt.matmul(a, b).array().shape == (0, 4)
    # K == 0: result is all zeros
    a = srt.Tensor(shape=[3, 0], dtype=np.float32)
    b = srt.Tensor(shape=[0, 4], dtype=np.float32)
    assert np.array_equal(srt.matmul(a, b).array(), np.zeros((3, 4), np.float32))


# ---- operands of 1 Gi elements and more (byte offsets beyond 32 bits) ---------------------------------
def _periodic(block, reps, axis):
    """`reps` copies of `block` along `axis`: a > 4 GB operand whose product is known from one block."""
    return np.ascontiguousarray(np.concatenate([block] * reps, axis=axis))


@pytest.mark.parametrize("case", ["nn_big_a", "nt_big_w", "tn_big_a", "skinny_big_w"])
def test_bf16_operands_beyond_4_gib_bit_exact(case):
    """An operand of 2.15 Gi bf16 elements (4.3 GB).  Where halves of M or N bring it within the 256 x 256
    kernels' 32-bit offsets the call runs in pieces; an m-contiguous A whose k walk alone is out of reach
    runs on the 128 x 128 tiles with 64-bit addressing.  Sparse {-1, 0, 1} operands: exact in any order;
    the big operand repeats a 1152-row block (4.5 tiles, so no piece boundary falls on a block boundary)."""
    r = H.rng(400)
    P, reps, K = 1152, 57, 32768                 # 57 x 1152 = 65664 rows
    big0 = (r.integers(-1, 2, (P, K)) * (r.random((P, K)) < 0.25)).astype(np.float32)
    small_rows = 8 if case == "skinny_big_w" else 512
    small = (r.integers(-1, 2, (small_rows, K)) * (r.random((small_rows, K)) < 0.25)).astype(np.float32)
    block = big0.astype(np.float64) @ small.astype(np.float64).T          # [P, small_rows], exact integers
    if case == "nn_big_a":      # A [65664, K] . B [K, 512]
        a, b, ta, tb = _periodic(H.encode(big0, H.BF16), reps, 0), H.encode(np.ascontiguousarray(small.T), H.BF16), False, False
        # (each half: 130 tiles and K = 32768 -- the tail-sharing form, two parts per tile)
        want, kernel = np.concatenate([block] * reps, 0), "mfma_256x256_m16_k64_tail/pieces"
    elif case == "tn_big_a":    # A stored [K, 65664], transposed
        a, b, ta, tb = _periodic(H.encode(np.ascontiguousarray(big0.T), H.BF16), reps, 1), H.encode(np.ascontiguousarray(small.T), H.BF16), True, False
        want, kernel = np.concatenate([block] * reps, 0), "mfma_128x128"
    else:                       # x [512 or 8, K] . W [65664, K]^T
        a, b, ta, tb = H.encode(small, H.BF16), _periodic(H.encode(big0, H.BF16), reps, 0), False, True
        want = np.concatenate([block.T] * reps, 1)
        # (each half of N: 258 tiles -- a whole round, and the two left over cut along k)
        kernel = "skinny/pieces" if case == "skinny_big_w" else "mfma_256x256_m16_k64_tail/pieces"
    assert max(a.size, b.size) > 2 ** 31
    got = gpu_matmul(a, b, ta, tb, want_kernel=kernel)
    assert np.array_equal(got, H.encode(want.astype(np.float32), H.BF16))


def test_bf16_batches_beyond_reach_run_in_pieces_bit_exact():
    """72 batches of 2048 x 8192 (1.2 Gi elements of A): the batch is halved until a piece is within reach;
    every batch must land in its own slab of the result.  Bias and ReLU go with every piece."""
    r = H.rng(401)
    nb, M, N, K = 72, 2048, 2048, 8192
    a0 = (r.integers(-1, 2, (3, M, K)) * (r.random((3, M, K)) < 0.25)).astype(np.float32)
    b0 = (r.integers(-1, 2, (3, K, N)) * (r.random((3, K, N)) < 0.25)).astype(np.float32)
    bias = r.integers(-4, 5, N).astype(np.float32)
    a = np.ascontiguousarray(np.concatenate([H.encode(a0, H.BF16)] * (nb // 3), 0))
    b = np.ascontiguousarray(np.concatenate([H.encode(b0, H.BF16)] * (nb // 3), 0))
    at, bt = srt.Tensor(a), srt.Tensor(b)
    out = srt.Tensor(shape=[nb, M, N], dtype=a.dtype)
    assert query_kernel(at, False, bt, False, out) == "mfma_256x256_m16_k64/pieces"
    srt.current_queue().matmul(at, False, bt, False, out, bias=srt.Tensor(H.encode(bias, H.BF16)),
                               activation=srt.ActivationType.relu)
    block = np.maximum(a0.astype(np.float64) @ b0.astype(np.float64) + bias, 0.0)
    want = H.encode(np.concatenate([block] * (nb // 3), 0).astype(np.float32), H.BF16)
    assert np.array_equal(out.array(), want)


def test_bias_follows_the_pieces_along_n():
    """x . W^T + bias with a W of 65664 x 16384 (1 Gi elements and 128 columns more): the pieces along N take
    their own part of the bias."""
    r = H.rng(402)
    P, reps, K, M = 1152, 57, 16384, 300
    w0 = (r.integers(-1, 2, (P, K)) * (r.random((P, K)) < 0.25)).astype(np.float32)
    x = (r.integers(-1, 2, (M, K)) * (r.random((M, K)) < 0.25)).astype(np.float32)
    bias = r.integers(-64, 65, P * reps).astype(np.float32)
    xt, wt = srt.Tensor(H.encode(x, H.BF16)), srt.Tensor(_periodic(H.encode(w0, H.BF16), reps, 0))
    out = srt.Tensor(shape=[M, P * reps], dtype=np.uint16)
    assert query_kernel(xt, False, wt, True, out).endswith("/pieces")
    srt.current_queue().matmul(xt, False, wt, True, out, bias=srt.Tensor(H.encode(bias, H.BF16)),
                               activation=srt.ActivationType.identity)
    block = x.astype(np.float64) @ w0.astype(np.float64).T
    want = np.concatenate([block] * reps, 1) + bias
    assert np.array_equal(out.array(), H.encode(want.astype(np.float32), H.BF16))


def test_fp32_operand_beyond_4_gib_vs_exact():
    """fp32 A of 33408 x 32768 (4.4 GB): the fp32 kernels address with 64-bit offsets."""
    r = H.rng(403)
    P, reps, K, N = 1152, 29, 32768, 256
    a0 = (r.integers(-2, 3, (P, K)) * (r.random((P, K)) < 0.25)).astype(np.float32)
    b = (r.integers(-2, 3, (K, N)) * (r.random((K, N)) < 0.25)).astype(np.float32)
    got = gpu_matmul(_periodic(a0, reps, 0), b)
    block = (a0.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, np.concatenate([block] * reps, 0))


# ---- fused sigmoid / tanh / elu near zero -----------------------------------------------------------
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("act", [srt.ActivationType.sigmoid, srt.ActivationType.tanh, srt.ActivationType.elu])
@pytest.mark.parametrize("plan,M,N", [(None, 64, 96), ("mfma_256x256_m16", 512, 512), ("mfma_256x256", 512, 512)])
def test_fused_transcendentals_keep_their_digits_near_zero(act, dt, plan, M, N, tmp_path):
    """Pre-activations from 1e-7 to 0.4 in magnitude, both signs (K = 8 with a single non-zero term, so the
    accumulator is exact): the fused epilogues work in fp32 with the hardware exponential (sigmoid, elu) or a
    quotient of polynomials (tanh); a closed form that cancels near 0 -- (e^2x - 1) / (e^2x + 1), exp(x) - 1 --
    would lose its digits here.  Every result must be within two rounding steps of the stored type, relative."""
    K = 8
    mags = np.logspace(-7, -0.4, N) * np.where(np.arange(N) % 2, -1.0, 1.0)
    x = np.zeros((M, K), np.float32)
    x[:, 0] = np.exp2(-(np.arange(M) % 12)).astype(np.float32)          # row scales, exact powers of two
    w = np.zeros((K, N), np.float32)
    w[0] = mags
    xs, ws = H.encode(x, dt), H.encode(w, dt)
    if plan is not None:
        pin_plan_for_shape(tmp_path, plan, dt, M, N, K)
    xt, wt = srt.Tensor(xs), srt.Tensor(ws)
    out = srt.Tensor(shape=[M, N], dtype=xs.dtype)
    srt.current_queue().matmul(xt, False, wt, False, out, activation=act, coef=1.0)
    if plan is not None:
        assert query_kernel(xt, False, wt, False, out) == plan
    got = H.decode(out.array()).astype(np.float64)
    pre = H.decode(xs)[:, :1].astype(np.float64) * H.decode(ws)[:1].astype(np.float64)     # exact in fp32
    want = {srt.ActivationType.sigmoid: lambda v: 1.0 / (1.0 + np.exp(-v)),
            srt.ActivationType.tanh: np.tanh,
            srt.ActivationType.elu: lambda v: np.where(v > 0, v, np.expm1(v))}[act](pre)
    floor = 2.0 ** -24 if dt == H.F16 else 1e-30          # a half's subnormal step
    assert np.all(np.abs(got - want) <= 2 * H.ULP[dt] * np.abs(want) + floor)
    srt.PlanCache.clear()


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_problems_through_the_librarys_own_choice_bit_exact(seed):
    """Widely random problems -- element type, layout, batch (own or shared right operand), extents drawn
    log-uniformly with and without alignment, bias, relu / clipped relu -- run on whatever kernel the library
    picks by itself.  Operands are small integers, so every sum is exact in fp32 and the stored result must
    equal the exact one rounded once, bit for bit.  The case is named before it runs."""
    g = np.random.default_rng(seed)
    q = srt.current_queue()
    seen = set()

    def logu(lo, hi):
        return int(np.exp(g.uniform(np.log(lo), np.log(hi + 1))))

    for case in range(250):
        dt = (H.F32, H.BF16, H.F16)[int(g.integers(0, 3))]
        ta, tb = bool(g.integers(0, 2)), bool(g.integers(0, 2))
        batch = int(g.choice([1, 1, 1, 2, 3, 7]))
        M, N, K = logu(1, 3000), logu(1, 3000), logu(1, 4096)
        if g.random() < 0.5:
            M, N, K = max(8, M // 8 * 8), max(8, N // 8 * 8), max(8, K // 8 * 8)
        if g.random() < 0.4:
            K = max(64, K // 64 * 64)
        if g.random() < 0.15:
            M = int(g.integers(1, 65))
        if M * N * K * batch > 3e9:
            continue
        with_bias = bool(g.integers(0, 2))
        act = (srt.ActivationType.identity, srt.ActivationType.relu, srt.ActivationType.clippedRelu)[int(g.integers(0, 3))]
        shared_b = batch > 1 and g.random() < 0.3
        what = (seed, case, dt, ta, tb, batch, M, N, K, with_bias, act, shared_b)
        sa = (K, M) if ta else (M, K)
        sb = (N, K) if tb else (K, N)
        a = g.integers(-2, 3, (batch,) + sa).astype(np.float32)
        b = g.integers(-2, 3, ((1,) if shared_b else (batch,)) + sb).astype(np.float32)
        bias = g.integers(-3, 4, N).astype(np.float32)
        exact = (a.transpose(0, 2, 1) if ta else a).astype(np.float64) @ (b.transpose(0, 2, 1) if tb else b).astype(np.float64)
        if with_bias:
            exact = exact + bias[None, None, :]
        if act != srt.ActivationType.identity:
            exact = np.maximum(exact, 0.0)
        if act == srt.ActivationType.clippedRelu:
            exact = np.minimum(exact, 6.0)
        want = H.encode(exact.astype(np.float32), dt)
        if batch == 1:
            at, bt = srt.Tensor(H.encode(a[0], dt)), srt.Tensor(H.encode(b[0], dt))
            out = srt.Tensor(shape=[M, N], dtype=at.dtype)
            want = want[0]
        else:
            at = srt.Tensor(H.encode(a, dt))
            bt = srt.Tensor.repeating(srt.Tensor(H.encode(b[0], dt)), (batch,) + sb) if shared_b else srt.Tensor(H.encode(b, dt))
            out = srt.Tensor(shape=[batch, M, N], dtype=at.dtype)
        seen.add(query_kernel(at, ta, bt, tb, out))
        q.matmul(at, ta, bt, tb, out, bias=srt.Tensor(H.encode(bias, dt)) if with_bias else None, activation=act, coef=6.0)
        assert np.array_equal(out.array().view(np.uint8), want.view(np.uint8)), what
    assert len(seen) >= 5, seen


@pytest.mark.parametrize("dt,M,N,K,ta,tb", [
    (H.BF16, 520, 776, 1024, False, False), (H.BF16, 1024, 4096, 4096, False, True), (H.BF16, 2048, 4096, 2048, False, False),
    (H.BF16, 1024, 8192, 512, True, False), (H.BF16, 3072, 1536, 8192, False, True), (H.BF16, 512, 1024, 4096, False, True),
    (H.BF16, 8, 1000, 520, False, True), (H.BF16, 8, 1096, 264, False, False), (H.F16, 200, 265, 72, False, False),
    (H.F16, 264, 328, 256, True, True), (H.F32, 8, 1000, 520, False, True), (H.F32, 8, 1096, 264, False, False),
    (H.F32, 512, 512, 512, False, False), (H.F32, 1024, 1024, 1024, False, False), (H.F32, 200, 264, 72, True, False),
    (H.F32, 512, 2048, 4096, False, True), (H.F32, 64, 2048, 4096, False, False)])
def test_nan_and_inf_stay_in_their_rows_on_the_librarys_own_choice(dt, M, N, K, ta, tb):
    """One NaN and one infinity in A (B all positive): row 5 of the result is NaN, row 7 is +inf, and every other element
    is the exact product -- a tile-wide or wave-wide shortcut in an encoder or an epilogue must not let a special value
    leak into a neighbour's row, whichever kernel the library picks for the shape."""
    g = H.rng(900 + M + K)
    a = g.integers(-2, 3, (M, K)).astype(np.float32)
    b = g.integers(1, 4, (K, N)).astype(np.float32)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    a[5, 1] = np.nan
    a[7, 2] = np.inf
    a_st = H.encode(np.ascontiguousarray(a.T) if ta else a, dt)
    b_st = H.encode(np.ascontiguousarray(b.T) if tb else b, dt)
    at, bt = srt.Tensor(a_st), srt.Tensor(b_st)
    out = srt.Tensor(shape=[M, N], dtype=at.dtype)
    kernel = query_kernel(at, ta, bt, tb, out)
    srt.current_queue().matmul(at, ta, bt, tb, out)
    got = out.array()
    dec = H.decode(got).astype(np.float64)
    assert np.all(np.isnan(dec[5])), kernel
    assert np.all(np.isposinf(dec[7])), kernel
    if dt == H.BF16:
        assert np.all(got[5] == 0x7FFF), kernel          # the reference codec's NaN (platform/common/BFloat16.swift:53-80)
    rest = np.ones(M, bool)
    rest[[5, 7]] = False
    want = H.encode(exact.astype(np.float32), dt)
    assert np.array_equal(got[rest].view(np.uint8), want[rest].view(np.uint8)), kernel


@pytest.mark.parametrize("M,N,K,tb", [(64, 64, 64, False), (200, 264, 72, False), (520, 776, 1024, False), (8, 1000, 520, True),
                                      (1024, 1024, 1024, False), (2048, 4096, 512, False), (4096, 4096, 512, False),
                                      (512, 1024, 4096, True)])
@pytest.mark.parametrize("dt,scale_a,scale_b", [
    (H.F16, 2.0 ** -24, 2.0 ** 6),       # subnormal halves in A, normal results
    (H.F16, 2.0 ** -12, 2.0 ** -12),     # results among the subnormal halves
    (H.F32, 2.0 ** -149, 2.0 ** 60),     # subnormal floats in A
    (H.F32, 2.0 ** -100, 2.0 ** -49),    # products and sums among the subnormal floats
    (H.BF16, 2.0 ** -133, 2.0 ** 100),   # subnormal bfloat16s in A
    (H.BF16, 2.0 ** -100, 2.0 ** -33)])  # sums that are subnormal in the fp32 accumulator and in the result
def test_subnormal_operands_and_results_are_kept(dt, scale_a, scale_b, M, N, K, tb):
    """The reference's CPU loops run with gradual underflow (Swift Float / Float16 arithmetic): small integers times a
    power of two that puts the operands, the products or the sums among the subnormals must give the exact scaled integer
    product -- no flush to zero on the way into the matrix cores, in their accumulators or in the stored result --
    whichever kernel the library picks."""
    g = H.rng(950 + M + K)
    a = g.integers(-2, 3, (M, K)).astype(np.float64) * scale_a
    b = g.integers(-2, 3, (K, N)).astype(np.float64) * scale_b
    exact = a @ b
    a_st = H.encode(a.astype(np.float32), dt)
    b_st = H.encode(np.ascontiguousarray(b.T if tb else b).astype(np.float32), dt)
    assert np.array_equal(H.decode(a_st).astype(np.float64), a) and np.count_nonzero(exact) > exact.size // 2
    at, bt = srt.Tensor(a_st), srt.Tensor(b_st)
    out = srt.Tensor(shape=[M, N], dtype=at.dtype)
    kernel = query_kernel(at, False, bt, tb, out)
    srt.current_queue().matmul(at, False, bt, tb, out)
    want = H.encode(exact.astype(np.float32), dt)
    assert np.array_equal(out.array().view(np.uint8), want.view(np.uint8)), kernel


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_random_operand_and_result_views_through_the_librarys_own_choice(seed):
    """As the random-problem test, with every tensor a view: row (or, in column-major order, column) pitches wider than the
    extent by nothing, a multiple of eight or an odd count, first elements at aligned and unaligned offsets, batches
    lying apart with gaps or -- for an operand -- repeated with stride 0, all of it inside buffers that hold a sentinel
    elsewhere.  Pitches and alignment decide which kernels qualify; the result must be exact inside its view and the rest
    of its buffer untouched, whichever kernel that leaves."""
    from numpy.lib.stride_tricks import as_strided
    g = np.random.default_rng(seed)
    q = srt.current_queue()
    seen = set()

    def logu(lo, hi):
        return int(np.exp(g.uniform(np.log(lo), np.log(hi + 1))))

    def strided(rows, cols, batch, col_major, may_repeat, aligned):
        unit = 8 if aligned else 1
        pad = int(g.choice([0, 0, 8, 24] if aligned else [0, 1, 3, 8, 13]))
        lead, other = (rows, cols) if col_major else (cols, rows)         # contiguous extent, strided extent
        pitch = lead + pad
        offset = int(g.integers(0, 4)) * unit
        matrix = pitch * other
        bstride = 0 if (may_repeat and batch > 1 and g.random() < 0.3) else matrix + int(g.integers(0, 3)) * pitch
        size = offset + (batch - 1) * bstride + matrix + 8
        strides2 = [1, pitch] if col_major else [pitch, 1]
        return offset, ([bstride] + strides2) if batch > 1 else strides2, size

    for case in range(150):
        dt = (H.F32, H.BF16, H.F16)[int(g.integers(0, 3))]
        ta, tb = bool(g.integers(0, 2)), bool(g.integers(0, 2))
        batch = int(g.choice([1, 1, 2, 4]))
        aligned = g.random() < 0.6
        M, N, K = logu(1, 600), logu(1, 600), logu(1, 2100)
        if aligned:
            M, N, K = max(8, M // 8 * 8), max(8, N // 8 * 8), max(8, K // 8 * 8)
        if g.random() < 0.3:
            K = max(64, K // 64 * 64)
        col_major = g.random() < 0.25
        order = srt.Order.col if col_major else srt.Order.row
        lead = [batch] if batch > 1 else []
        tensors, dense = [], []
        for (rows, cols, repeat) in [((K, M) if ta else (M, K)) + (True,), ((N, K) if tb else (K, N)) + (True,)]:
            off, strides, size = strided(rows, cols, batch, col_major, repeat, aligned)
            flat = H.encode(np.full(size, 77.0, np.float32), dt)
            view = as_strided(flat[off:], lead + [rows, cols], [s * flat.itemsize for s in strides])
            shape_written = [1 if s == 0 else e for e, s in zip(lead + [rows, cols], strides)]
            values = g.integers(-2, 3, shape_written).astype(np.float32)
            view[tuple(slice(0, e) for e in shape_written)] = H.encode(values, dt)
            base = srt.Tensor(flat)
            tensors.append(srt.Tensor(shape=lead + [rows, cols], order=order, _storage=base.storage, _offset=off, _strides=strides))
            full = np.broadcast_to(values, lead + [rows, cols]).astype(np.float64)
            dense.append(full.reshape(batch, rows, cols))
        a64 = dense[0].transpose(0, 2, 1) if ta else dense[0]
        b64 = dense[1].transpose(0, 2, 1) if tb else dense[1]
        bias = g.integers(-3, 4, N).astype(np.float32)
        with_bias = bool(g.integers(0, 2))
        relu = bool(g.integers(0, 2))
        exact = a64 @ b64 + (bias[None, None, :] if with_bias else 0.0)
        if relu:
            exact = np.maximum(exact, 0.0)
        off, strides, size = strided(M, N, batch, col_major, False, aligned)
        sentinel = H.encode(np.full(size, 12345.0, np.float32), dt)
        obase = srt.Tensor(sentinel.copy())
        out = srt.Tensor(shape=lead + [M, N], order=order, _storage=obase.storage, _offset=off, _strides=strides)
        want_flat = sentinel.copy()
        as_strided(want_flat[off:], lead + [M, N], [s * want_flat.itemsize for s in strides])[...] = \
            H.encode(exact.astype(np.float32), dt).reshape(lead + [M, N])
        what = (seed, case, dt, ta, tb, batch, M, N, K, col_major, aligned, [t.strides for t in tensors], strides, off, with_bias, relu)
        kernel = query_kernel(tensors[0], ta, tensors[1], tb, out)
        seen.add(kernel)
        q.matmul(tensors[0], ta, tensors[1], tb, out, bias=srt.Tensor(H.encode(bias, dt)) if with_bias else None,
                 activation=srt.ActivationType.relu if relu else srt.ActivationType.identity)
        assert np.array_equal(obase.array().view(np.uint8), want_flat.view(np.uint8)), what + (kernel,)
    assert len(seen) >= 4, seen
