"""GPU parity tests of the path the headline benchmark times: the persistent 256 x 256 kernels with
several tiles per workgroup, whole k stages and the k loop running across tile boundaries (the next
tile's first stages are requested while the current tile's last ones are multiplied).

Integer-valued operands in [-3, 3] make every partial sum exact in fp32 for K up to 1.8 M, so the
result is bit-exact whatever the summation order: each pinned plan must reproduce, bit for bit,
(a) the exact product on sampled rows and columns that cross every tile (float64 matmul of small
integers is exact), and (b) over the WHOLE result, what the 128 x 128 kernel computes -- a kernel
with no persistent grid, no ring and no cross-tile state, itself checked against the oracle at
smaller sizes.
"""
import ctypes

import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native
from tests import helpers as H

pytestmark = pytest.mark.gpu

LAYOUTS = [(False, False), (False, True), (True, False), (True, True)]


@pytest.fixture(autouse=True)
def clean_plan_cache():
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


def pin(tmp_path, plan, dt, M, N, K, ta, tb, bias=False, act=srt.ActivationType.identity, batch=1):
    layout = (2 if ta else 1) | (4 if tb else 8) | 16 | 64
    f = tmp_path / "plan.txt"
    # the call's own epilogue key, and the plain one the kernel query looks up
    keys = {(1 if bias else 0) | (int(act) << 1), int(srt.ActivationType.identity) << 1}
    f.write_text("".join(f"{dt} {M} {N} {K} {batch} {layout} {e} {plan}\n" for e in sorted(keys)))
    srt.PlanCache.clear()
    srt.PlanCache.load(f)


_operands = {}


def integer_operands(dt, shape, seed):
    """One storage array of integers in [-3, 3] per (type, shape, seed), kept on the device."""
    key = (dt, tuple(shape), seed)
    if key not in _operands:
        vals = H.rng(seed).integers(-3, 4, tuple(shape)).astype(np.float32)
        t = srt.Tensor(H.encode(vals, dt))
        t.device_read(srt.current_queue())
        _operands[key] = (vals, t)
    return _operands[key]


def sample(extent, count, salt):
    """`count` indices spread over [0, extent): every 256-wide tile is crossed, at varying offsets inside it."""
    step = max(1, extent // count)
    idx = (np.arange(count) * step + (np.arange(count) * salt) % step) % extent
    return np.unique(idx)


def run_pinned(tmp_path, plan, dt, a_t, ta, b_t, tb, M, N, K, bias=None, act=srt.ActivationType.identity):
    pin(tmp_path, plan, dt, M, N, K, ta, tb, bias=bias is not None, act=act)
    out = srt.Tensor(shape=[M, N], dtype=H.NP_STORAGE[dt])
    assert query_kernel(a_t, ta, b_t, tb, out) == plan
    srt.current_queue().matmul(a_t, ta, b_t, tb, out, bias=bias, activation=act)
    return out.array()


def check_plan(tmp_path, plan, dt, M, N, K, ta, tb, with_bias_relu=False):
    a_vals, a_t = integer_operands(dt, (K, M) if ta else (M, K), seed=41)
    b_vals, b_t = integer_operands(dt, (N, K) if tb else (K, N), seed=42)
    bias_vals = bias_t = None
    act = srt.ActivationType.identity
    if with_bias_relu:
        bias_vals, bias_t = integer_operands(dt, (N,), seed=43)
        act = srt.ActivationType.relu
    got = run_pinned(tmp_path, plan, dt, a_t, ta, b_t, tb, M, N, K, bias=bias_t, act=act)
    # (a) sampled rows and columns against the exact product
    a64 = (a_vals.T if ta else a_vals).astype(np.float64)
    b64 = (b_vals.T if tb else b_vals).astype(np.float64)
    rows, cols = sample(M, 64, 37), sample(N, 64, 53)

    def finish(x, bias_part):
        if with_bias_relu:
            x = np.maximum(x + bias_part, 0.0)
        return H.encode(x.astype(np.float32), dt)

    want_rows = finish(a64[rows] @ b64, None if bias_vals is None else bias_vals[None, :].astype(np.float64))
    want_cols = finish(a64 @ b64[:, cols], None if bias_vals is None else bias_vals[None, cols].astype(np.float64))
    assert np.array_equal(got[rows].view(np.uint16), want_rows.view(np.uint16)), (plan, "rows")
    assert np.array_equal(got[:, cols].view(np.uint16), want_cols.view(np.uint16)), (plan, "columns")
    # (b) every element against the 128 x 128 kernel
    ref = run_pinned(tmp_path, "mfma_128x128", dt, a_t, ta, b_t, tb, M, N, K, bias=bias_t, act=act)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), (plan, "whole result")
    return got


def plans_for(ta, tb, K):
    plans = ["mfma_256x256_m16_k64", "mfma_256x256_m16", "mfma_256x256"]
    if K % 128 == 0 and K >= 256:
        plans.append("mfma_128x128_m16_k128")    # the quarter tile: whole 128-deep units, at least two
    if not ta and tb:
        plans.append("mfma_256x256_k64")    # two k-contiguous operands
    if not ta:
        plans.append("mfma_128x256_m16")    # k-contiguous A
        plans.append("mfma_128x256_m16_k64")
    else:
        plans.append("mfma_256x128_m16_k64")    # the half tile of the other A layouts
    return plans


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_headline_shape_integer_bit_exact(dt, ta, tb, tmp_path):
    """8192^3: 1024 tiles = 4 per workgroup, 256 whole stages, per-XCD k rotation with a transposed lhs."""
    for plan in plans_for(ta, tb, 8192):
        check_plan(tmp_path, plan, dt, 8192, 8192, 8192, ta, tb)


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_ragged_round_integer_bit_exact(dt, ta, tb, tmp_path):
    """4608 x 4608 x 2048: 324 tiles on 256 workgroups (a second, ragged round; the grid is evened to 168),
    64 whole stages; and 4400 x 4360 x 320: edge tiles in M and N, ten whole stages = five 64-deep units."""
    for plan in plans_for(ta, tb, 2048):
        check_plan(tmp_path, plan, dt, 4608, 4608, 2048, ta, tb)
    for plan in plans_for(ta, tb, 320):
        check_plan(tmp_path, plan, dt, 4400, 4360, 320, ta, tb)


# ---- the 128 x 128 quarter tile (128-deep units) on small pinned shapes ---------------------------------------
QUARTER = "mfma_128x128_m16_k128"


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_quarter_tile_integer_bit_exact_and_random_vs_fp64(dt, ta, tb, tmp_path):
    """Every staging layout; the shortest admissible k loops (two and three units: every request beyond the first fill
    belongs to the next tile), an odd number of units, ragged edges in M and N (a last tile of 8 rows, of 8 columns), one
    tile and several per workgroup (1225 tiles), fewer tiles than workgroups; then random operands against the fp64 product."""
    r = H.rng(311)
    for (M, N, K) in [(256, 384, 512), (1000, 520, 640), (2048, 2056, 896), (4400, 4360, 512), (136, 128, 1152),
                      (4400, 4360, 256), (2056, 2048, 384), (136, 72, 256)]:
        pin(tmp_path, QUARTER, dt, M, N, K, ta, tb)
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        at, bt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt))
        out = srt.Tensor(shape=[M, N], dtype=H.NP_STORAGE[dt])
        assert query_kernel(at, ta, bt, tb, out) == QUARTER
        srt.current_queue().matmul(at, ta, bt, tb, out)
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    M, N, K = 2040, 2056, 1024
    pin(tmp_path, QUARTER, dt, M, N, K, ta, tb)
    a_st = H.encode((r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32), dt)
    b_st = H.encode(r.standard_normal((N, K) if tb else (K, N)).astype(np.float32), dt)
    out = srt.matmul(srt.Tensor(a_st), srt.Tensor(b_st), transposed_lhs=ta, transposed_rhs=tb).array()
    a64, b64 = H.to64(a_st), H.to64(b_st)
    c64 = (a64.T if ta else a64) @ (b64.T if tb else b64)
    assert H.max_norm_rel(H.decode(out), c64) <= H.TOL[dt]
    absprod = np.abs(a64.T if ta else a64) @ np.abs(b64.T if tb else b64)
    assert H.elementwise_excess(H.decode(out), c64, absprod, dt, K) <= 1.0


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("act", list(srt.ActivationType))
@pytest.mark.parametrize("tw", [False, True])
def test_quarter_tile_epilogues_vs_oracle(act, dt, tw, tmp_path):
    """y = act(x . W + b) and act(x . W^T + b): every activation through the fused epilogue, ragged M / N edges."""
    from oracle import srt_oracle as ora
    r = H.rng(29)
    M, N, K = 1100, 1032, 512
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((N, K) if tw else (K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    pin(tmp_path, QUARTER, dt, M, N, K, False, tw, bias=True, act=act)
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    assert query_kernel(xt, False, wt, tw, out) == QUARTER
    srt.current_queue().matmul(xt, False, wt, tw, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 131), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=tw,
                                      acc=ora.ACC_F32, fused=True))
    tol = {H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got[rows] - want) <= tol * np.maximum(np.abs(want), 1.0))


def test_quarter_tile_broadcast_weight_and_column_major():
    """The heuristic's own choice on a batch against one shared weight (batch stride 0, the descriptor built by hand) and on
    a column-major call with bias and relu (computed as the transposed problem, bias per row of what the kernel stores)."""
    srt.PlanCache.clear()
    r = H.rng(37)
    q = srt.current_queue()
    for dt in (H.BF16, H.F16):
        B_, M, N, K = 3, 520, 392, 512
        a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
        w = r.integers(-3, 4, (K, N)).astype(np.float32)
        at, wt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(w, dt))
        out = srt.Tensor(shape=[B_, M, N], dtype=H.NP_STORAGE[dt])
        ad, k1 = at.descriptor()
        bd, k2 = native.make_descriptor(native.REAL16F if dt == H.F16 else native.REAL16BF, (B_, K, N), (0, N, 1), native.ORDER_ROW)
        od, k3 = out.descriptor()
        buf = ctypes.create_string_buffer(64)
        native.check(native.lib().srtMatmulQueryKernel(ctypes.byref(ad), 0, ctypes.byref(bd), 0, ctypes.byref(od), at.device_read(q),
                                                       wt.device_read(q), out.device_read(q), buf, 64))
        assert buf.value.decode() == QUARTER
        native.check(native.lib().srtMatmul(at.device_read(q), ctypes.byref(ad), 0, wt.device_read(q), ctypes.byref(bd), 0,
                                            out.device_read_write(q), ctypes.byref(od), q.stream))
        exact = H.encode((a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), dt)
        assert np.array_equal(out.array().view(np.uint16), exact.view(np.uint16)), dt
        M2, N2, K2 = 776, 520, 640
        x = r.integers(-3, 4, (M2, K2)).astype(np.float32)
        w2 = r.integers(-3, 4, (K2, N2)).astype(np.float32)
        b2 = r.integers(-30, 31, N2).astype(np.float32)
        xc, wc = srt.Tensor(H.encode(x, dt), order=srt.Order.col), srt.Tensor(H.encode(w2, dt), order=srt.Order.col)
        yc = srt.Dense(wc, srt.Tensor(H.encode(b2, dt)), srt.ActivationType.relu)(xc)
        assert yc.order == srt.Order.col and query_kernel(xc, False, wc, False, yc) == QUARTER
        want = np.maximum(x.astype(np.float64) @ w2.astype(np.float64) + b2.astype(np.float64)[None, :], 0)
        assert np.array_equal(yc.array().view(np.uint16), H.encode(want.astype(np.float32), dt).view(np.uint16)), dt


def test_quarter_tile_batched_and_nan(tmp_path):
    """Strided batch (tiles of several batches per workgroup), and NaN / inf results encoded as the reference's codec does."""
    r = H.rng(31)
    B_, M, N, K = 5, 1024, 1032, 640
    a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (B_, K, N)).astype(np.float32)
    pin(tmp_path, QUARTER, H.BF16, M, N, K, False, False, batch=B_)
    at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
    out = srt.matmul(at, wt)
    assert query_kernel(at, False, wt, False, out) == QUARTER
    assert np.array_equal(out.array(), H.encode((a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), H.BF16))
    M = N = 768
    K = 512
    a = np.zeros((M, K), np.float32)
    w = np.zeros((K, N), np.float32)
    a[:, 0] = 1.0
    w[0, :] = 2.0
    a[5, 1] = np.nan
    a[7, 1] = np.inf
    w[1, :] = 1.0
    pin(tmp_path, QUARTER, H.BF16, M, N, K, False, False)
    at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
    out = srt.matmul(at, wt)
    assert query_kernel(at, False, wt, False, out) == QUARTER
    got = out.array()
    assert np.all(got[5] == 0x7FFF) and np.all(got[7] == 0x7F80)
    assert np.all(got[6] == H.encode(np.array([2.0], np.float32), H.BF16)[0])


# ---- the 64-deep form of the 16x16x32 kernel on small pinned shapes ------------------------------------------
DEEP = "mfma_256x256_m16_k64"


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_k64_m16_integer_bit_exact_and_random_vs_fp64(dt, ta, tb, tmp_path):
    """Every staging layout; the shortest admissible k loop (four units), an odd number of units, ragged edges
    in M and N, one tile and several per workgroup; then random operands against the fp64 product."""
    from oracle import srt_oracle as ora
    r = H.rng(301)
    for (M, N, K) in [(512, 512, 256), (1000, 520, 320), (2048, 2056, 448), (4400, 4360, 576)]:
        pin(tmp_path, DEEP, dt, M, N, K, ta, tb)
        a = r.integers(-3, 4, (K, M) if ta else (M, K)).astype(np.float32)
        b = r.integers(-3, 4, (N, K) if tb else (K, N)).astype(np.float32)
        at, bt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt))
        out = srt.Tensor(shape=[M, N], dtype=H.NP_STORAGE[dt])
        assert query_kernel(at, ta, bt, tb, out) == DEEP
        srt.current_queue().matmul(at, ta, bt, tb, out)
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(out.array().view(np.uint16), H.encode(exact.astype(np.float32), dt).view(np.uint16)), (M, N, K)
    M, N, K = 2040, 2056, 512
    pin(tmp_path, DEEP, dt, M, N, K, ta, tb)
    a_st = H.encode((r.standard_normal((K, M) if ta else (M, K)) / np.sqrt(K)).astype(np.float32), dt)
    b_st = H.encode(r.standard_normal((N, K) if tb else (K, N)).astype(np.float32), dt)
    out = srt.matmul(srt.Tensor(a_st), srt.Tensor(b_st), transposed_lhs=ta, transposed_rhs=tb).array()
    a64, b64 = H.to64(a_st), H.to64(b_st)
    c64 = (a64.T if ta else a64) @ (b64.T if tb else b64)
    assert H.max_norm_rel(H.decode(out), c64) <= H.TOL[dt]
    absprod = np.abs(a64.T if ta else a64) @ np.abs(b64.T if tb else b64)
    assert H.elementwise_excess(H.decode(out), c64, absprod, dt, K) <= 1.0


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("act", list(srt.ActivationType))
@pytest.mark.parametrize("tw", [False, True])
def test_k64_m16_epilogues_vs_oracle(act, dt, tw, tmp_path):
    """y = act(x . W + b) and act(x . W^T + b): every activation through the fused epilogue, ragged M / N edges."""
    from oracle import srt_oracle as ora
    r = H.rng(23)
    M, N, K = 2100, 2056, 256
    x = H.encode(r.standard_normal((M, K)).astype(np.float32), dt)
    w = H.encode((r.standard_normal((N, K) if tw else (K, N)) / 8).astype(np.float32), dt)
    b = H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), dt)
    coef = 0.75
    pin(tmp_path, DEEP, dt, M, N, K, False, tw, bias=True, act=act)
    xt, wt, bt = srt.Tensor(x), srt.Tensor(w), srt.Tensor(b)
    out = srt.Tensor(shape=[M, N], dtype=x.dtype)
    assert query_kernel(xt, False, wt, tw, out) == DEEP
    srt.current_queue().matmul(xt, False, wt, tw, out, bias=bt, activation=act, coef=coef)
    got = H.decode(out.array())
    rows = np.concatenate([np.arange(0, M, 131), [M - 1]])
    want = H.decode(ora.dense_forward(np.ascontiguousarray(x[rows]), w, b, int(act), coef=coef, transpose_w=tw,
                                      acc=ora.ACC_F32, fused=True))
    tol = {H.F16: 2.0 ** -10, H.BF16: 2.0 ** -7}[dt]
    assert np.all(np.abs(got[rows] - want) <= tol * np.maximum(np.abs(want), 1.0))


def test_k64_m16_batched_column_major_and_nan(tmp_path):
    """Strided batch (tiles of several batches per workgroup), a column-major call (computed as the transposed
    problem, bias per row), and NaN / inf results encoded as the reference's codec does."""
    r = H.rng(24)
    B_, M, N, K = 3, 1024, 1032, 320
    a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (B_, K, N)).astype(np.float32)
    pin(tmp_path, DEEP, H.BF16, M, N, K, False, False, batch=B_)
    at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
    out = srt.matmul(at, wt)
    assert query_kernel(at, False, wt, False, out) == DEEP
    assert np.array_equal(out.array(), H.encode((a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), H.BF16))
    M = N = 1536
    K = 256
    a = np.zeros((M, K), np.float32)
    w = np.zeros((K, N), np.float32)
    a[:, 0] = 1.0
    w[0, :] = 2.0
    a[5, 1] = np.nan
    a[7, 1] = np.inf
    w[1, :] = 1.0
    pin(tmp_path, DEEP, H.BF16, M, N, K, False, False)
    at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
    out = srt.matmul(at, wt)
    assert query_kernel(at, False, wt, False, out) == DEEP
    got = out.array()
    assert np.all(got[5] == 0x7FFF) and np.all(got[7] == 0x7F80)
    assert np.all(got[6] == H.encode(np.array([2.0], np.float32), H.BF16)[0])


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
def test_column_major_dense_through_the_flipped_kernels(dt):
    """Column-major operands and result: the call is computed as the transposed problem, whose A is k-contiguous and
    whose B is n-contiguous -- the layout the 64-deep kernel and its tail-sharing form run flipped -- with the bias
    running along the rows of what the kernel stores.  Integer operands and bias, relu, ragged edges: bit-exact."""
    srt.PlanCache.clear()
    r = H.rng(808)
    relu = srt.ActivationType.relu
    for (M, N, K, want) in [(2056, 4088, 512, DEEP), (3072, 1536, 8192, TAIL), (3064, 1528, 8192, TAIL), (1016, 4088, 4096, QUARTER)]:
        a = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (K, N)).astype(np.float32)
        bias = r.integers(-40, 41, N).astype(np.float32)
        at = srt.Tensor(H.encode(a, dt), order=srt.Order.col)
        wt = srt.Tensor(H.encode(w, dt), order=srt.Order.col)
        bt = srt.Tensor(H.encode(bias, dt))
        out = srt.Tensor(shape=[M, N], dtype=at.dtype, order=srt.Order.col)
        assert query_kernel(at, False, wt, False, out) == want, (M, N, K)
        srt.current_queue().matmul(at, False, wt, False, out, bias=bt, activation=relu)
        exact = np.maximum(a.astype(np.float64) @ w.astype(np.float64) + bias, 0)   # (integers: exact in fp64)
        assert np.array_equal(out.array(), H.encode(exact.astype(np.float32), dt)), (M, N, K)


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
def test_dense_shape_bias_relu_integer_bit_exact(dt, tmp_path):
    """The Dense configuration's shape, 4096 x 11008 x 4096 with an integer bias and relu: 688 tiles run as
    three even rounds of 232 workgroups."""
    for plan in ("mfma_256x256_m16_k64", "mfma_256x256_m16", "mfma_256x256"):
        got = check_plan(tmp_path, plan, dt, 4096, 11008, 4096, False, False, with_bias_relu=True)
        assert np.all(H.decode(got) >= 0.0)


def test_heuristic_takes_the_checked_kernels():
    """The shapes above are run by the kernels checked above when nothing is pinned."""
    a = srt.Tensor(shape=[8192, 8192], dtype=np.uint16)
    out = srt.Tensor(shape=[8192, 8192], dtype=np.uint16)
    assert query_kernel(a, False, a, False, out) == "mfma_256x256_m16_k64"
    assert query_kernel(a, True, a, False, out) == "mfma_256x256_m16_k64"
    x = srt.Tensor(shape=[4096, 4096], dtype=np.uint16)
    w = srt.Tensor(shape=[4096, 11008], dtype=np.uint16)
    y = srt.Tensor(shape=[4096, 11008], dtype=np.uint16)
    assert query_kernel(x, False, w, False, y) == "mfma_256x256_m16_k64"


# ---- the tail-sharing form of the 64-deep kernel ------------------------------------------------------------
TAIL = "mfma_256x256_m16_k64_tail"


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_tail_sharing_integer_bit_exact(dt, ta, tb, tmp_path):
    """Tiles left over after the whole rounds, cut along k and added up by whichever piece ends last:
    2048 x 4096 x 2048 -- 128 tiles and no whole round, two parts per tile (5 + 3 quads);
    4096 x 5120 x 2048 -- one whole round, then 64 tiles in three parts (4 + 2 + 2);
    4400 x 4360 x 2048 -- ragged edges in M and N, 68 tiles left over (not a multiple of 8), three parts."""
    for (M, N, K) in [(2048, 4096, 2048), (4096, 5120, 2048), (4400, 4360, 2048)]:
        check_plan(tmp_path, TAIL, dt, M, N, K, ta, tb)


def test_tail_sharing_dense_shape_bias_relu(tmp_path):
    """4096 x 11008 x 4096 with bias and relu: two whole rounds, then 176 tiles cut 14 + 2 quads, the short
    parts taken three at a time by 64 further workgroups."""
    got = check_plan(tmp_path, TAIL, H.BF16, 4096, 11008, 4096, False, False, with_bias_relu=True)
    assert np.all(H.decode(got) >= 0.0)


def test_tail_sharing_batched_clipped_and_repeatable(tmp_path):
    """A strided batch (96 tiles over three batches, two parts each), the clipped-relu epilogue on random
    operands against the plain kernel (the parts' sums are added in another order: one rounding step of the
    result type apart at most), and the same bits on every run, whichever piece happened to add up."""
    r = H.rng(77)
    B_, M, N, K = 3, 1024, 2048, 1024
    a = r.integers(-3, 4, (B_, M, K)).astype(np.float32)
    w = r.integers(-3, 4, (B_, K, N)).astype(np.float32)
    pin(tmp_path, TAIL, H.BF16, M, N, K, False, False, batch=B_)
    at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
    out = srt.matmul(at, wt)
    assert query_kernel(at, False, wt, False, out) == TAIL
    assert np.array_equal(out.array(), H.encode((a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32), H.BF16))

    M, N, K = 2048, 4096, 4096
    x = srt.Tensor(H.encode((r.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32), H.BF16))
    wt = srt.Tensor(H.encode(r.standard_normal((K, N)).astype(np.float32), H.BF16))
    bt = srt.Tensor(H.encode(r.uniform(-0.5, 0.5, N).astype(np.float32), H.BF16))
    act = srt.ActivationType.clippedRelu
    runs = {}
    for plan in (TAIL, DEEP):
        pin(tmp_path, plan, H.BF16, M, N, K, False, False, bias=True, act=act)
        out = srt.Tensor(shape=[M, N], dtype=np.uint16)
        assert query_kernel(x, False, wt, False, out) == plan
        runs[plan] = []
        for _ in range(3 if plan == TAIL else 1):
            srt.current_queue().matmul(x, False, wt, False, out, bias=bt, activation=act, coef=0.75)
            runs[plan].append(out.array().copy())
    assert np.array_equal(runs[TAIL][0], runs[TAIL][1]) and np.array_equal(runs[TAIL][0], runs[TAIL][2])
    tail, plain = H.decode(runs[TAIL][0]), H.decode(runs[DEEP][0])
    assert np.all(np.abs(tail - plain) <= 2.0 ** -7 * np.maximum(np.abs(plain), 2.0 ** -7))
    assert np.count_nonzero(runs[TAIL][0] != runs[DEEP][0]) < 0.01 * M * N
    assert tail.max() == 0.75 and tail.min() == 0.0


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_few_tile_batches_with_long_k(ta, tb, tmp_path):
    """A batch has no split-K pass.  The heuristic gives its few tiles to the 128 x 128 quarter tile (one round of them);
    pinned, the tail-sharing kernel cuts every tile of the launch along k (three parts each).  The batches have their own
    operands and the tiles have ragged edges: integer operands, bit-exact in every layout, both ways."""
    r = H.rng(515)
    for (B_, M, N, K, dt) in [(4, 256, 256, 4096, H.BF16), (5, 200, 520, 4096, H.F16), (16, 136, 144, 8192, H.BF16)]:
        a = r.integers(-2, 3, (B_, K, M) if ta else (B_, M, K)).astype(np.float32)
        w = r.integers(-2, 3, (B_, N, K) if tb else (B_, K, N)).astype(np.float32)
        at, wt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(w, dt))
        am = np.swapaxes(a, 1, 2) if ta else a
        wm = np.swapaxes(w, 1, 2) if tb else w
        exact = am.astype(np.float64) @ wm.astype(np.float64)   # (small integers: exact in fp64)
        for plan in (QUARTER, TAIL):
            srt.PlanCache.clear()
            if plan == TAIL:
                pin(tmp_path, TAIL, dt, M, N, K, ta, tb, batch=B_)
            out = srt.matmul(at, wt, ta, tb)
            assert query_kernel(at, ta, wt, tb, out) == plan, (B_, M, N, K)
            assert np.array_equal(out.array(), H.encode(exact.astype(np.float32), dt)), (plan, B_, M, N, K)
    srt.PlanCache.clear()


def test_tail_sharing_on_two_queues_at_once():
    """Two queues launch tail-sharing matmuls of different shapes back to back without waiting for each other:
    every launch has its own partial sums and flags (stream-ordered workspace, a launch-unique flag value), so
    the results are the ones each queue gets alone -- bit for bit, on integer operands the exact product."""
    srt.PlanCache.clear()
    p = srt.HipPlatform.local()
    q0, q1 = p.devices[1].queues[0], p.devices[1].queues[1]
    r = H.rng(616)
    jobs = []
    for (q, (M, N, K)) in [(q0, (3072, 3072, 4096)), (q1, (3072, 1536, 8192))]:
        a = r.integers(-2, 3, (M, K)).astype(np.float32)
        w = r.integers(-2, 3, (N, K)).astype(np.float32)
        at, wt = srt.Tensor(H.encode(a, H.BF16)), srt.Tensor(H.encode(w, H.BF16))
        outs = [srt.Tensor(shape=[M, N], dtype=np.uint16) for _ in range(6)]
        assert query_kernel(at, False, wt, True, outs[0]) == TAIL, (M, N, K)
        at.device_read(q); wt.device_read(q)
        want = H.encode((a.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32), H.BF16)
        jobs.append((q, at, wt, outs, want))
    q0.wait_for_completion(); q1.wait_for_completion()
    for i in range(6):
        for (q, at, wt, outs, _) in jobs:
            q.matmul(at, False, wt, True, outs[i])
    for (q, _, _, outs, want) in jobs:
        q.wait_for_completion()
        for o in outs:
            assert np.array_equal(o.array(), want)


def test_tail_sharing_every_way_of_cutting(tmp_path):
    """Left-over counts that reach every branch of the cutting rule -- three parts, two parts, one short part
    taken two, three and four at a time, counts that are not multiples of 8, a single left-over tile, with and
    without whole rounds before them -- on ragged M and N, in rotating layouts and both types: bit-exact against
    the 128 x 128 kernel over the whole result."""
    r = H.rng(911)
    # (tiles along M, tiles along N, batch, K): left over = tiles mod 256
    cases = [(1, 1, 1, 1792),      # 1 tile: three parts (7 quads: 4 + 2 + 1)
             (1, 7, 1, 1024),      # 7: a 4-quad tile is too short for three parts -> two (3 + 1)
             (3, 3, 1, 2304),      # 9: three parts (5 + 2 + 2)
             (5, 16, 1, 1792),     # 80: three parts, every compute unit but 16 at work
             (2, 43, 1, 1024),     # 86: two parts
             (3, 43, 1, 1792),     # 129: two parts (6 + 1), the short one taken two at a time
             (9, 19, 1, 2560),     # 171: (9 + 1) three at a time
             (4, 11, 4, 2560),     # 176 over four batches: three at a time
             (8, 25, 1, 3328),     # 200: (12 + 1) four at a time
             (16, 17, 1, 1024),    # 272 = a whole round + 16
             (11, 31, 1, 1280)]    # 341 = a whole round + 85
    for i, (tm, tn, batch, K) in enumerate(cases):
        dt = (H.BF16, H.F16)[i % 2]
        ta, tb = LAYOUTS[i % 4]
        M = tm * 256 - int(r.integers(0, 31)) * 8
        N = tn * 256 - int(r.integers(0, 31)) * 8
        a = r.integers(-3, 4, (batch, K, M) if ta else (batch, M, K)).astype(np.float32)
        b = r.integers(-3, 4, (batch, N, K) if tb else (batch, K, N)).astype(np.float32)
        at, bt = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt))
        got = {}
        for plan in (TAIL, "mfma_128x128"):
            pin(tmp_path, plan, dt, M, N, K, ta, tb, batch=batch)
            out = srt.Tensor(shape=[batch, M, N], dtype=H.NP_STORAGE[dt])
            assert query_kernel(at, ta, bt, tb, out) == plan, (plan, tm, tn, batch, K)
            srt.current_queue().matmul(at, ta, bt, tb, out)
            got[plan] = out.array().copy()
        assert np.array_equal(got[TAIL].view(np.uint16), got["mfma_128x128"].view(np.uint16)), (tm, tn, batch, K, ta, tb)
        # and a sampled row of each batch against the exact product
        for z in range(batch):
            row = int(r.integers(0, M))
            a_row = (a[z][:, row] if ta else a[z][row]).astype(np.float64)
            b_mat = (b[z].T if tb else b[z]).astype(np.float64)
            want = H.encode((a_row @ b_mat).astype(np.float32), dt)
            assert np.array_equal(got[TAIL][z, row].view(np.uint16), want.view(np.uint16)), (tm, tn, z, row)


def test_tail_sharing_is_refused_where_it_does_not_apply(tmp_path):
    """No tiles left over, k not in whole quads, or too few quads to cut: a pinned tail-sharing plan is ignored
    and the heuristic's kernel runs."""
    def kernel_for(M, N, K):
        pin(tmp_path, TAIL, H.BF16, M, N, K, False, False)
        a = srt.Tensor(shape=[M, K], dtype=np.uint16)
        b = srt.Tensor(shape=[K, N], dtype=np.uint16)
        out = srt.Tensor(shape=[M, N], dtype=np.uint16)
        return query_kernel(a, False, b, False, out)
    assert kernel_for(2048, 4096, 2048) == TAIL
    assert kernel_for(4096, 4096, 2048) != TAIL      # 256 tiles: nothing left over
    assert kernel_for(2048, 4096, 2048 + 64) != TAIL  # k not a multiple of 256
    assert kernel_for(2048, 4096, 512) != TAIL        # two quads: too short to cut


# ---- the reference's batched known answers on the device, bf16 included -----------------------------------
@pytest.mark.parametrize("dt", [H.F32, H.F16, H.BF16])
def test_reference_kat_batched_and_right_batched(kats, dt):
    """test_AlgebraicField.swift:572-597 (batched) through the codec -- values up to 275 are not all bf16
    numbers -- and the right-batched form: one lhs matrix against a batch (batch stride 0)."""
    k = kats["matmul_batched"]
    a = H.encode(np.arange(12, dtype=np.float32).reshape(k["a_arange_shape"]), dt)
    b = H.encode(np.arange(16, dtype=np.float32).reshape(k["b_arange_shape"]), dt)
    got = srt.matmul(srt.Tensor(a), srt.Tensor(b)).array()
    assert np.array_equal(got.view(np.uint8), H.encode(np.array(k["c"], np.float32), dt).view(np.uint8))
    kr = kats["matmul_right_batched"]
    a2 = srt.Tensor(H.encode(np.arange(6, dtype=np.float32).reshape(3, 2), dt))
    a3 = srt.Tensor.repeating(a2, (2, 3, 2))
    assert a3.strides[0] == 0
    got = srt.matmul(a3, srt.Tensor(b)).array()
    assert np.array_equal(got.view(np.uint8), H.encode(np.array(kr["c"], np.float32), dt).view(np.uint8))


# ---- the split form: whole rounds of 256 x 256 tiles, then one round of 192-wide tiles ----------------------------
@pytest.mark.parametrize("dt", [H.BF16, H.F16])
@pytest.mark.parametrize("ta,tb", LAYOUTS)
def test_split_form_integer_bit_exact(dt, ta, tb, tmp_path):
    """4096 x 11008 (16 x 43 tiles = 2.69 rounds of 256 workgroups: 8192 columns in whole tiles, 2816 in 16 narrow tiles
    of 176 per row of tiles) with bias + relu, K = 512; 2000 x 13000 x 256 (8 x 51 tiles = 1.59 rounds: 32 narrow tiles of
    152 per row, ragged last row of tiles); 4104 x 10480 x 320 (17 rows of tiles, 15 narrow tiles of 192 per row: 255 of the 256
    workgroups take one)."""
    check_plan(tmp_path, "mfma_256x256_m16_k64_split", dt, 4096, 11008, 512, ta, tb, with_bias_relu=True)
    check_plan(tmp_path, "mfma_256x256_m16_k64_split", dt, 2000, 13000, 256, ta, tb)
    check_plan(tmp_path, "mfma_256x256_m16_k64_split", dt, 4104, 10480, 320, ta, tb, with_bias_relu=True)


def test_split_form_is_offered_for_the_dense_shape_and_refused_where_it_does_not_apply(tmp_path):
    a = srt.Tensor(shape=[4096, 4096], dtype=np.uint16)
    b = srt.Tensor(shape=[4096, 11008], dtype=np.uint16)
    out = srt.Tensor(shape=[4096, 11008], dtype=np.uint16)
    assert query_kernel(a, False, b, False, out) == "mfma_256x256_m16_k64"      # the heuristic never takes it (a wash)
    pin(tmp_path, "mfma_256x256_m16_k64_split", H.BF16, 4096, 11008, 4096, False, False)
    assert query_kernel(a, False, b, False, out) == "mfma_256x256_m16_k64_split"
    # 8192^3 has no ragged round; 4096 x 10240 leaves exactly half a round (a 128-wide tile's case); a batch has no split form
    for (M, N, K, batch) in [(8192, 8192, 8192, 1), (4096, 10240, 4096, 1), (1024, 2752, 256, 4)]:
        lead = [batch] if batch > 1 else []
        a = srt.Tensor(shape=lead + [M, K], dtype=np.uint16)
        b = srt.Tensor(shape=lead + [K, N], dtype=np.uint16)
        out = srt.Tensor(shape=lead + [M, N], dtype=np.uint16)
        pin(tmp_path, "mfma_256x256_m16_k64_split", H.BF16, M, N, K, False, False, batch=batch)
        assert query_kernel(a, False, b, False, out) != "mfma_256x256_m16_k64_split", (M, N, K, batch)


# ---- operands that alias the result -------------------------------------------------------------------
def test_result_overlapping_an_operand_is_refused():
    q = srt.current_queue()
    buf = srt.Tensor(np.zeros((64, 64), np.float32))
    other = srt.Tensor(np.zeros((32, 32), np.float32))
    a, out = buf[0:32, 0:32], buf[16:48, 0:32]      # spans overlap
    with pytest.raises(native.SrtError) as e:
        q.matmul(a, False, other, False, out)
    assert e.value.status == native.ERROR_INVALID_VALUE
    with pytest.raises(native.SrtError):
        q.matmul(other, False, a, False, out)
    # disjoint row blocks of one buffer are fine
    lo, hi = buf[0:32, :], buf[32:64, :]
    w = srt.Tensor(np.eye(64, dtype=np.float32))
    q.matmul(lo, False, w, False, hi)


def test_column_slices_and_interleaved_batches_of_one_buffer_are_accepted():
    # storage spans overlap, yet a common pitch proves the views apart: operand, bias and result as column
    # slices of one wide row-major buffer, and operand and result as alternate batches of one buffer
    q = srt.current_queue()
    r = H.rng(91)
    wide = r.integers(-3, 4, (48, 96)).astype(np.float32)
    buf = srt.Tensor(wide.copy())
    w = r.integers(-3, 4, (32, 32)).astype(np.float32)
    a, out = buf[:, 0:32], buf[:, 64:96]
    bias = srt.Tensor(shape=[32], order=buf.order, _storage=buf.storage, _offset=buf.offset + 32, _strides=[1])
    q.matmul(a, False, srt.Tensor(w), False, out, bias=bias)
    got = buf.array()
    assert np.array_equal(got[:, 64:96], wide[:, 0:32] @ w + wide[0, 32:64])
    assert np.array_equal(got[:, 0:64], wide[:, 0:64])            # the rest of the buffer is untouched
    both = r.integers(-3, 4, (6, 16, 24)).astype(np.float32)
    buf3 = srt.Tensor(both.copy())
    w3 = r.integers(-3, 4, (3, 24, 24)).astype(np.float32)
    q.matmul(buf3[0::2], False, srt.Tensor(w3), False, buf3[1::2])
    got = buf3.array()
    assert np.array_equal(got[1::2], both[0::2] @ w3)
    assert np.array_equal(got[0::2], both[0::2])
    # even against odd columns of one buffer (the element pitch of 2 proves them apart)
    eo = r.integers(-3, 4, (16, 64)).astype(np.float32)
    buf2 = srt.Tensor(eo.copy())
    w2 = r.integers(-3, 4, (32, 32)).astype(np.float32)
    q.matmul(buf2[:, 0::2], False, srt.Tensor(w2), False, buf2[:, 1::2])
    got = buf2.array()
    assert np.array_equal(got[:, 1::2], eo[:, 0::2] @ w2)
    assert np.array_equal(got[:, 0::2], eo[:, 0::2])
