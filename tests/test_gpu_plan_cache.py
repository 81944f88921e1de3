"""GPU tests of the plan / tune cache: srtMatmulTune measures every kernel plan a problem qualifies
for, records the fastest, and later matmuls with the same key run it; every plan computes the same
product (bit-exact on integer-valued inputs)."""
import ctypes

import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native
from tests import helpers as H
from tests.test_gpu_matmul import query_kernel

pytestmark = pytest.mark.gpu

PLANS_16 = {"mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail", "mfma_256x256_m16_k64_split", "mfma_256x256", "mfma_256x256_k64", "mfma_256x256_m16", "mfma_256x256_splitk", "mfma_128x256_m16", "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_128x128_m16_k128", "mfma_128x128", "mfma_64x64", "mfma_128x128_any", "mfma_64x64_any", "skinny", "generic"}
PLANS_32 = {"f32_mfma_64x64", "f32_mfma_splitk", "f32_mfma_128x128_parts", "f32_mfma_128x128_ring", "f32_mfma_64x128_ring", "f32_mfma_64x64_ring", "generic"}


@pytest.fixture(autouse=True)
def clean_cache():
    srt.PlanCache.clear()
    yield
    srt.PlanCache.clear()


def int_operands(seed, m, k, n, dt, ta=False, tb=False):
    g = H.rng(seed)
    a = H.encode(g.integers(-4, 5, (k, m) if ta else (m, k)).astype(np.float32), dt)
    b = H.encode(g.integers(-4, 5, (n, k) if tb else (k, n)).astype(np.float32), dt)
    return a, b


@pytest.mark.parametrize("dt,m,k,n,ta,tb", [(H.BF16, 1024, 64, 1024, False, False), (H.F16, 512, 32, 768, True, False),
                                            (H.BF16, 8, 128, 2048, False, True), (H.F32, 256, 64, 256, False, False)])
def test_tune_records_a_plan_and_later_calls_use_it(dt, m, k, n, ta, tb):
    a_st, b_st = int_operands(41, m, k, n, dt, ta, tb)
    a, b = srt.Tensor(a_st), srt.Tensor(b_st)
    q = srt.current_queue()
    # integer sums below 2^24 are exact in fp32 in any order; the store rounds once to the element type
    exact = H.to64(a_st.T if ta else a_st) @ H.to64(b_st.T if tb else b_st)
    want = H.to64(H.encode(exact.astype(np.float32), dt))
    heuristic = srt.matmul(a, b, ta, tb)
    assert np.array_equal(H.to64(heuristic.array()), want)
    out = srt.Tensor(shape=[m, n], dtype=a.dtype)
    chosen = q.tune_matmul(a, ta, b, tb, out)
    assert chosen in (PLANS_32 if dt == H.F32 else PLANS_16)
    assert srt.PlanCache.count() == 1
    assert np.array_equal(H.to64(out.array()), want)                            # `out` was left by the chosen plan
    name = query_kernel(a, ta, b, tb, out)
    assert name == chosen or (name == "f32_mfma" and chosen.startswith("f32_mfma"))
    again = srt.matmul(a, b, ta, tb)                                            # runs the cached plan
    assert np.array_equal(H.to64(again.array()), want)
    # another shape is not affected
    a2, b2 = int_operands(42, m, k + 8, n, dt, ta, tb)
    srt.matmul(srt.Tensor(a2), srt.Tensor(b2), ta, tb)
    assert srt.PlanCache.count() == 1


def test_every_plan_is_the_same_function(tmp_path):
    """Forces each 16-bit plan in turn through a hand-written cache file and compares the products:
    bit-exact on integers, and within one bf16 rounding of each other on normal data."""
    m = k = n = 512
    a_st, b_st = int_operands(43, m, k, n, H.BF16)
    g = H.rng(44)
    ar = H.encode((g.standard_normal((m, k)) / np.sqrt(k)).astype(np.float32), H.BF16)
    br = H.encode(g.standard_normal((k, n)).astype(np.float32), H.BF16)
    want = H.to64(H.encode((H.to64(a_st) @ H.to64(b_st)).astype(np.float32), H.BF16))
    results = {}
    for plan in ("mfma_256x256", "mfma_128x128", "mfma_64x64", "mfma_128x128_any", "mfma_64x64_any", "generic"):
        f = tmp_path / f"{plan}.txt"
        f.write_text(f"14 {m} {n} {k} 1 89 10 {plan}\n")
        srt.PlanCache.clear()
        srt.PlanCache.load(f)
        a, b = srt.Tensor(a_st), srt.Tensor(b_st)
        c = srt.matmul(a, b)
        assert query_kernel(a, False, b, False, c) == plan
        assert np.array_equal(H.to64(c.array()), want), plan
        results[plan] = H.to64(srt.matmul(srt.Tensor(ar), srt.Tensor(br)).array())
    c64 = H.to64(ar) @ H.to64(br)
    for plan, r in results.items():
        assert H.max_norm_rel(r, c64) <= H.TOL[H.BF16], plan
        assert np.max(np.abs(r - results["generic"]) / (np.abs(c64) + 1e-3)) <= 2 ** -6, plan


ALL_PLANS_16 = ("mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail", "mfma_256x256_m16_k64_split", "mfma_256x256_m16", "mfma_256x256", "mfma_256x256_k64", "mfma_256x256_splitk", "mfma_128x256_m16", "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_128x128_m16_k128", "mfma_128x128",
                "mfma_64x64", "mfma_128x128_any", "mfma_64x64_any", "skinny", "generic")


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_every_qualifying_plan_bit_exact(seed, tmp_path):
    """Random shapes, layouts, element types, bias and activation: every plan that accepts the problem
    (asked through the cache, answered by the kernel query) must give the exact integer result.  A
    plan that claims a problem it mishandles -- a ragged edge, a k tail, a split that does not divide
    -- shows up here whatever the heuristic would have chosen."""
    g = H.rng(5000 + seed)
    ran = set()
    for case in range(7):
        dt = (H.BF16, H.F16)[int(g.integers(0, 2))]
        ta, tb = bool(g.integers(0, 2)), bool(g.integers(0, 2))
        M = int(g.choice([8, 24, 32, 200, 264, 520, 1032]))
        N = int(g.choice([8, 40, 256, 264, 776, 1288]))
        K = int(g.choice([8, 64, 72, 200, 1024, 2048, 4096]))
        with_bias = bool(g.integers(0, 2))
        act = (srt.ActivationType.identity, srt.ActivationType.relu)[int(g.integers(0, 2))]
        a = g.integers(-2, 3, (K, M) if ta else (M, K)).astype(np.float32)
        b = g.integers(-2, 3, (N, K) if tb else (K, N)).astype(np.float32)
        bias = g.integers(-3, 4, N).astype(np.float32)
        exact = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        if with_bias:
            exact = exact + bias[None, :]
        if act == srt.ActivationType.relu:
            exact = np.maximum(exact, 0.0)
        want = H.encode(exact.astype(np.float32), dt).view(np.uint16)
        at, bt, biast = srt.Tensor(H.encode(a, dt)), srt.Tensor(H.encode(b, dt)), srt.Tensor(H.encode(bias, dt))
        layout = (2 if ta else 1) | (4 if tb else 8) | 16 | 64
        for plan in ALL_PLANS_16:
            # the query has no epilogue argument: ask with the plain key, run with the real one
            for epilogue in {10, (1 if with_bias else 0) | (int(act) << 1)}:
                f = tmp_path / "p.txt"
                f.write_text(f"{dt} {M} {N} {K} 1 {layout} {epilogue} {plan}\n")
                srt.PlanCache.load(f)
            out = srt.Tensor(shape=[M, N], dtype=at.dtype)
            if query_kernel(at, ta, bt, tb, out) != plan:
                srt.PlanCache.clear()
                continue
            srt.current_queue().matmul(at, ta, bt, tb, out, bias=biast if with_bias else None, activation=act)
            assert np.array_equal(out.array().view(np.uint16), want), (plan, dt, ta, tb, M, N, K, with_bias, act)
            ran.add(plan)
            srt.PlanCache.clear()
    print("plans exercised:", sorted(ran))
    assert "generic" in ran and len(ran) >= 3


def test_cached_plan_is_skipped_when_this_call_does_not_qualify(tmp_path):
    """Alignment is not part of the key: a view that starts off a 16-byte boundary with the same
    shape and layout class falls back to the heuristic (the kernel with element-wise staging) instead
    of the cached plan, whose 16-byte loads it does not qualify for."""
    m = k = n = 256
    f = tmp_path / "p.txt"
    f.write_text(f"14 {m} {n} {k} 1 89 10 mfma_64x64\n")
    srt.PlanCache.load(f)
    g = H.rng(45)
    big = H.encode(g.integers(-3, 4, (m, k + 8)).astype(np.float32), H.BF16)
    b_st = H.encode(g.integers(-3, 4, (k, n)).astype(np.float32), H.BF16)
    a_view = srt.Tensor(big)[:, 1:k + 1]                 # row pitch 264 (16-byte multiple), start misaligned by 2 bytes
    c = srt.matmul(a_view, srt.Tensor(b_st))
    assert query_kernel(a_view, False, srt.Tensor(b_st), False, c) == "mfma_64x64_any"
    exact = H.to64(big[:, 1:k + 1]) @ H.to64(b_st)
    assert np.array_equal(H.to64(c.array()), H.to64(H.encode(exact.astype(np.float32), H.BF16)))


def test_tune_errors():
    q = srt.current_queue()
    L = native.lib()
    a = srt.Tensor(np.zeros((4, 8), np.float32))
    b = srt.Tensor(np.zeros((9, 4), np.float32))
    o = srt.Tensor(shape=[4, 4], dtype=np.float32)
    ad, k1 = a.descriptor()
    bd, k2 = b.descriptor()
    od, k3 = o.descriptor()
    name = ctypes.create_string_buffer(16)
    assert L.srtMatmulTune(a.device_read(q), ctypes.byref(ad), 0, b.device_read(q), ctypes.byref(bd), 0, None, None, 5,
                           0.0, o.device_read_write(q), ctypes.byref(od), q.stream, name, 16) == native.ERROR_INVALID_VALUE
    ad.type = bd.type = od.type = native.REAL64F
    bd2, k4 = native.make_descriptor(native.REAL64F, (8, 4), (4, 1), native.ORDER_ROW)
    assert L.srtMatmulTune(a.device_read(q), ctypes.byref(ad), 0, b.device_read(q), ctypes.byref(bd2), 0, None, None, 5,
                           0.0, o.device_read_write(q), ctypes.byref(od), q.stream, name, 16) == native.ERROR_NOT_SUPPORTED
    assert srt.PlanCache.count() == 0
