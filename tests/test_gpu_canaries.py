"""Out-of-bounds write canaries for every store path of the library.

Results (and operands) are views inside larger buffers that are filled with a sentinel bit pattern before the
call; afterwards every byte outside the views must still hold it, and the views must hold the exact result.
The kernels store through staged 16-byte chunks on ragged edges and into strided views, so a store that runs
past an edge, into the gap between rows or into a neighbouring batch shows up here whatever the values are.
Every kernel plan is pinned in turn through the plan cache (as in test_gpu_plan_cache); the streaming kernel's
56-column tiles, the split-K reduction, the element-wise kernel's vector and scalar paths and the backward
epilogue have cases of their own."""
import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native
from tests import helpers as H
from tests.test_gpu_matmul import query_kernel

pytestmark = pytest.mark.gpu

SENTINEL = {np.dtype(np.uint16): 0x7B5A, np.dtype(np.float16): 0x7B5A, np.dtype(np.float32): 0x7B5A7B5A}
# a quiet NaN of each type: around an OPERAND it shows whether anything outside the view reaches a sum
# (a finite value times a padding zero vanishes, a NaN does not)
NAN_BITS = {np.dtype(np.uint16): 0x7FC0, np.dtype(np.float16): 0x7E00, np.dtype(np.float32): 0x7FC00000}

ALL_PLANS_16 = ("mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail", "mfma_256x256_m16_k64_split", "mfma_256x256_m16", "mfma_256x256", "mfma_256x256_k64",
                "mfma_256x256_splitk", "mfma_128x256_m16", "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_128x128_m16_k128", "mfma_128x128", "mfma_64x64", "mfma_128x128_any",
                "mfma_64x64_any", "skinny", "generic")
ALL_PLANS_32 = ("f32_mfma_64x64", "f32_mfma_splitk", "f32_mfma_128x128_parts", "f32_mfma_128x128_ring", "f32_mfma_64x128_ring", "f32_mfma_64x64_ring", "generic")


@pytest.fixture(autouse=True)
def clean_cache():
    srt.PlanCache.clear()
    yield
    srt.PlanCache.clear()


class Framed:
    """A `shape` view (rank 2 or 3) inside a larger buffer full of the sentinel: `top` rows above and below,
    `left` / `right` elements either side of every row, `between` whole sentinel matrices between batches."""

    def __init__(self, values, top=2, left=8, right=8, between=1, sentinel=None):
        values = np.asarray(values)
        sentinel = SENTINEL if sentinel is None else sentinel
        self.np_dtype = values.dtype
        self.bits = np.dtype(np.uint32) if values.dtype == np.float32 else np.dtype(np.uint16)
        shape = values.shape
        batch = shape[0] if len(shape) == 3 else 1
        rows, cols = shape[-2], shape[-1]
        self.rows, self.cols, self.batch = rows, cols, batch
        self.top, self.left = top, left
        self.step = 1 + between
        big = np.full((batch * self.step, rows + 2 * top, left + cols + right), sentinel[values.dtype], self.bits)
        body = values.reshape(batch, rows, cols).view(self.bits)
        big[::self.step, top:top + rows, left:left + cols] = body
        self.before = big.copy()
        self.tensor = srt.Tensor(big.view(values.dtype))
        v = self.tensor[::self.step, top:top + rows, left:left + cols]
        if len(shape) == 2:
            v = srt.Tensor(shape=[rows, cols], order=v.order, _storage=v.storage, _offset=v.offset, _strides=v.strides[1:])
        self.view = v

    def inside(self):
        got = self.tensor.array().view(self.bits)
        return got[::self.step, self.top:self.top + self.rows, self.left:self.left + self.cols]

    def assert_frame_untouched(self, what):
        got = self.tensor.array().view(self.bits).copy()
        want = self.before.copy()
        got[::self.step, self.top:self.top + self.rows, self.left:self.left + self.cols] = 0
        want[::self.step, self.top:self.top + self.rows, self.left:self.left + self.cols] = 0
        bad = np.argwhere(got != want)
        assert bad.size == 0, f"{what}: {len(bad)} elements outside the view were written, first at {bad[0].tolist()}"

    def assert_unchanged(self, what):
        assert np.array_equal(self.tensor.array().view(self.bits), self.before), f"{what}: an operand buffer was written"


def pin(tmp_path, dt, M, N, K, batch, layout, epilogues, plan):
    f = tmp_path / "p.txt"
    f.write_text("".join(f"{dt} {M} {N} {K} {batch} {layout} {e} {plan}\n" for e in epilogues))
    srt.PlanCache.load(f)


def run_matmul_case(tmp_path, dt, M, N, K, batch, ta, tb, plans, seed, left=8, right=8, with_bias=True, relu=True,
                    operand_sentinel=None):
    """Every plan of `plans` that takes the problem: exact result inside the views, sentinel everywhere else."""
    g = H.rng(seed)
    lead = (batch,) if batch > 1 else ()
    a = g.integers(-2, 3, lead + ((K, M) if ta else (M, K))).astype(np.float32)
    b = g.integers(-2, 3, lead + ((N, K) if tb else (K, N))).astype(np.float32)
    bias = g.integers(-3, 4, N).astype(np.float32)
    exact = np.swapaxes(a, -1, -2) if ta else a
    exact = exact.astype(np.float64) @ (np.swapaxes(b, -1, -2) if tb else b).astype(np.float64)
    if with_bias:
        exact = exact + bias
    if relu:
        exact = np.maximum(exact, 0.0)
    want = H.encode(exact.astype(np.float32), dt)
    act = srt.ActivationType.relu if relu else srt.ActivationType.identity
    fa = Framed(H.encode(a, dt), left=left, right=right, sentinel=operand_sentinel)
    fb = Framed(H.encode(b, dt), left=left, right=right, sentinel=operand_sentinel)
    fbias = Framed(H.encode(bias, dt).reshape(1, N), top=1, left=left, right=right, sentinel=operand_sentinel)
    bias_t = srt.Tensor(shape=[N], order=fbias.view.order, _storage=fbias.view.storage, _offset=fbias.view.offset, _strides=[1])
    aligned = all((left + x.shape[-1] + right) % 8 == 0 for x in (a, b)) and (left + N + right) % 8 == 0
    layout = (2 if ta else 1) | (4 if tb else 8) | 16 | (64 if aligned else 0)
    ran = []
    for plan in plans:
        fo = Framed(np.zeros(lead + (M, N), want.dtype), left=left, right=right)
        pin(tmp_path, dt, M, N, K, batch, layout, {10, (1 if with_bias else 0) | (int(act) << 1)}, plan)
        # (the query reports both fp32 tile plans under one family name)
        if query_kernel(fa.view, ta, fb.view, tb, fo.view) != ("f32_mfma" if plan.startswith("f32_mfma") else plan):
            srt.PlanCache.clear()
            continue
        srt.current_queue().matmul(fa.view, ta, fb.view, tb, fo.view, bias=bias_t if with_bias else None, activation=act)
        what = (plan, dt, M, N, K, batch, ta, tb, left, right)
        bits = fo.bits
        assert np.array_equal(fo.inside().reshape(want.shape), want.view(bits)), what
        fo.assert_frame_untouched(what)
        fa.assert_unchanged(what)
        fb.assert_unchanged(what)
        fbias.assert_unchanged(what)
        ran.append(plan)
        srt.PlanCache.clear()
    return ran


# ---- every 16-bit plan, ragged M and N, views with gaps ----------------------------------------------
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_every_16_bit_plan_keeps_inside_a_ragged_result_view(ta, tb, tmp_path):
    """520 x 776 x 1024: three rows and four columns of 256-wide tiles, the last of each ragged (8 and 8 wide), K in whole
    quads of 64-deep units (tail sharing: 12 tiles left over, two parts; split-K: two parts)."""
    ran = run_matmul_case(tmp_path, H.BF16, 520, 776, 1024, 1, ta, tb, ALL_PLANS_16, 700 + 2 * ta + tb)
    print("plans exercised:", ran)
    for must in ("mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail", "mfma_256x256_m16", "mfma_256x256", "mfma_256x256_splitk",
                 "mfma_128x128_m16_k128", "mfma_128x128", "mfma_64x64", "generic"):
        assert must in ran, must
    if not ta:
        assert "mfma_128x256_m16" in ran and "mfma_128x256_m16_k64" in ran
    else:
        assert "mfma_256x128_m16_k64" in ran
    if not ta and tb:
        assert "mfma_256x256_k64" in ran


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
def test_every_plan_keeps_inside_batched_views_with_gaps(dt, tmp_path):
    """Three batches of 264 x 328 x 256 whose matrices lie two matrices apart in every buffer (a sentinel matrix between
    neighbours), rows with sentinel columns either side."""
    for ta, tb in [(False, False), (True, True), (False, True)]:
        ran = run_matmul_case(tmp_path, dt, 264, 328, 256, 3, ta, tb, ALL_PLANS_16, 720 + 2 * ta + tb)
        assert "mfma_256x256_m16_k64" in ran and "mfma_64x64" in ran and "generic" in ran, ran


def test_quarter_tile_keeps_inside_small_and_batched_views(tmp_path):
    """The 128 x 128 tile on results much smaller than a tile (8 and 40 rows of an m-contiguous A, 72 columns), on ragged
    edges in both directions, and on batches whose matrices lie two apart with sentinel columns either side of every row."""
    Q = ("mfma_128x128_m16_k128",)
    for (M, N, K, batch, ta, tb) in [(8, 72, 512, 1, True, False), (40, 1096, 640, 1, True, True), (136, 200, 512, 1, False, False),
                                     (264, 328, 512, 3, False, True), (72, 136, 1024, 5, True, False)]:
        for dt in (H.BF16, H.F16):
            ran = run_matmul_case(tmp_path, dt, M, N, K, batch, ta, tb, Q, 730 + M + batch)
            assert ran == list(Q), (M, N, K, batch, ta, tb, dt)


def test_plans_for_unaligned_views_keep_inside(tmp_path):
    """N not a multiple of 8, odd row pitches and bases off a 16-byte boundary: the element-wise staging kernels
    and the generic kernel (the 16-byte store paths do not qualify and must not be chosen)."""
    for (M, N, K, left, right) in [(200, 265, 72, 3, 2), (130, 72, 136, 1, 4), (257, 129, 65, 8, 3)]:
        for ta, tb in [(False, False), (True, False), (False, True)]:
            ran = run_matmul_case(tmp_path, H.BF16, M, N, K, 1, ta, tb, ALL_PLANS_16, 740 + M, left=left, right=right)
            assert set(ran) <= {"mfma_128x128_any", "mfma_64x64_any", "generic"} and "generic" in ran, ran
            assert "mfma_64x64_any" in ran, ran


def test_streaming_kernel_keeps_inside_including_its_56_column_tiles(tmp_path):
    """M <= 64 against a k-contiguous weight; 32 x 14336 runs on 256 workgroups of 56 columns; 14344 leaves a last tile of
    8 columns; an n-contiguous weight streams 64 columns per workgroup."""
    for (M, N, K, tb) in [(32, 14336, 256, True), (32, 14344, 128, True), (24, 14328, 128, True), (8, 1000, 520, True),
                          (64, 14336, 128, True), (8, 1096, 264, False), (40, 2056, 128, False)]:
        ran = run_matmul_case(tmp_path, H.BF16, M, N, K, 1, False, tb, ("skinny",), 760 + M + N % 97)
        assert ran == ["skinny"], (M, N, K, tb)
    ran = run_matmul_case(tmp_path, H.F16, 16, 520, 136, 5, False, True, ("skinny",), 777)
    assert ran == ["skinny"]


def test_fp32_plans_keep_inside(tmp_path):
    for (M, N, K, batch, ta, tb) in [(200, 264, 72, 1, False, False), (130, 70, 33, 1, True, False), (96, 136, 64, 3, False, True)]:
        ran = run_matmul_case(tmp_path, H.F32, M, N, K, batch, ta, tb, ALL_PLANS_32, 780 + M, left=4, right=4)
        assert "generic" in ran and len(ran) >= 2, ran


def test_nothing_outside_an_operand_view_reaches_a_sum(tmp_path):
    """Operand and bias views framed by NaNs (rows above and below, columns either side of every row, whole NaN matrices
    between batches): the reference's loops never touch an element outside a view, so every result must still be the exact
    one.  A kernel that reads a k tail, a ragged row or a neighbouring batch past the view's edge and counts on the other
    operand's padding zero to cancel it fails here."""
    cases16 = [(520, 776, 1024, 1), (200, 264, 72, 1), (130, 136, 200, 1), (264, 328, 1032, 1), (264, 328, 256, 3), (72, 136, 1024, 5)]
    for dt in (H.BF16, H.F16):
        for (M, N, K, batch) in cases16:
            for ta, tb in [(False, False), (False, True), (True, False), (True, True)]:
                ran = run_matmul_case(tmp_path, dt, M, N, K, batch, ta, tb, ALL_PLANS_16, 800 + M + K, operand_sentinel=NAN_BITS)
                assert "generic" in ran and len(ran) >= 3, ran
    for (M, N, K, left, right) in [(200, 265, 72, 3, 2), (130, 72, 136, 1, 4), (257, 129, 65, 8, 3)]:
        for ta, tb in [(False, False), (True, False), (False, True), (True, True)]:
            ran = run_matmul_case(tmp_path, H.BF16, M, N, K, 1, ta, tb, ALL_PLANS_16, 820 + M, left=left, right=right,
                                  operand_sentinel=NAN_BITS)
            assert "mfma_64x64_any" in ran, ran
    for (M, N, K, tb) in [(32, 14336, 256, True), (24, 14328, 136, True), (8, 1000, 520, True), (8, 1096, 264, False), (40, 2056, 136, False)]:
        for dt in (H.BF16, H.F32):
            if dt == H.F32 and M > 32:
                continue          # the fp32 form streams at most 32 rows
            ran = run_matmul_case(tmp_path, dt, M, N, K, 1, False, tb, ("skinny",), 840 + M, left=8, right=8, operand_sentinel=NAN_BITS)
            assert ran == ["skinny"], (dt, M, N, K, tb)
    for (M, N, K, batch, ta, tb) in [(200, 264, 72, 1, False, False), (130, 70, 33, 1, True, False), (96, 136, 64, 3, False, True),
                                     (264, 392, 1096, 1, False, True), (520, 264, 2048, 1, True, True), (136, 1032, 516, 2, False, False)]:
        ran = run_matmul_case(tmp_path, H.F32, M, N, K, batch, ta, tb, ALL_PLANS_32, 860 + M, left=4, right=4, operand_sentinel=NAN_BITS)
        assert "generic" in ran and len(ran) >= 2, ran


def test_column_major_result_view_keeps_inside():
    """A column-major result is computed as the transposed product; its view inside a larger column-major buffer
    (sentinel rows above and below every column) must stay inside too."""
    g = H.rng(799)
    M, N, K = 264, 520, 256
    a = g.integers(-2, 3, (M, K)).astype(np.float32)
    b = g.integers(-2, 3, (K, N)).astype(np.float32)
    want = H.encode((a.astype(np.float64) @ b).astype(np.float32), H.BF16)
    # storage [N + 4 columns][M + 16 rows], the view starts 8 rows down and 2 columns in
    big = np.full((N + 4, M + 16), SENTINEL[np.dtype(np.uint16)], np.uint16)
    t = srt.Tensor(big)
    out = srt.Tensor(shape=[M, N], order=srt.Order.col, _storage=t.storage, _offset=2 * (M + 16) + 8, _strides=[1, M + 16])
    srt.current_queue().matmul(srt.Tensor(H.encode(a, H.BF16)), False, srt.Tensor(H.encode(b, H.BF16)), False, out)
    got = t.array()
    assert np.array_equal(got[2:2 + N, 8:8 + M].T, want)
    got[2:2 + N, 8:8 + M] = SENTINEL[np.dtype(np.uint16)]
    assert np.all(got == SENTINEL[np.dtype(np.uint16)])


# ---- element-wise kernel: vector path, scalar path, broadcast, conversion ---------------------------------
@pytest.mark.parametrize("dt", [H.BF16, H.F16, H.F32])
def test_elementwise_results_keep_inside_their_views(dt):
    g = H.rng(801)
    q = srt.current_queue()
    # (rows, cols, left, right): 16-byte vectors possible / impossible (odd extent, odd pitch, misaligned base)
    for (rows, cols, left, right) in [(37, 264, 8, 8), (37, 264, 8, 4), (37, 261, 8, 3), (5, 1000, 3, 5), (129, 8, 0, 8)]:
        x = g.integers(-6, 7, (rows, cols)).astype(np.float32)
        y = g.integers(1, 5, (rows, cols)).astype(np.float32)
        row = g.integers(-3, 4, (1, cols)).astype(np.float32)
        fx, fy, frow = Framed(H.encode(x, dt), left=left, right=right), Framed(H.encode(y, dt), left=left, right=right), \
            Framed(H.encode(row, dt), top=1, left=left, right=right)
        brow = srt.Tensor.repeating(frow.view, (rows, cols))
        cases = [("add", lambda o: q.add(fx.view, fy.view, o), x + y),
                 ("mul", lambda o: q.mul(fx.view, fy.view, o), x * y),
                 ("max", lambda o: q.max(fx.view, fy.view, o), np.maximum(x, y)),
                 ("add row", lambda o: q.add(fx.view, brow, o), x + row),
                 ("sub element", lambda o: q.subtract(fx.view, 2.0, o), x - 2.0),
                 ("neg", lambda o: q.neg(fx.view, o), -x),
                 ("copy", lambda o: q.copy(fx.view, o), x)]
        for name, call, exact in cases:
            fo = Framed(np.zeros((rows, cols), fx.np_dtype), left=left, right=right)
            call(fo.view)
            what = (name, dt, rows, cols, left, right)
            assert np.array_equal(fo.inside()[0], H.encode(exact, dt).view(fo.bits)), what
            fo.assert_frame_untouched(what)
        for f in (fx, fy, frow):
            f.assert_unchanged((dt, rows, cols))
        # conversion into another element type's view
        other = H.F32 if dt != H.F32 else H.BF16
        fo = Framed(H.encode(np.zeros((rows, cols), np.float32), other), left=left, right=right)
        q.copy(fx.view, fo.view)
        assert np.array_equal(fo.inside()[0], H.encode(x, other).view(fo.bits)), ("convert", dt, rows, cols)
        fo.assert_frame_untouched(("convert", dt, rows, cols, left, right))
        # transcendental results: only the frame is checked here (values have tests of their own)
        fo = Framed(np.zeros((rows, cols), fx.np_dtype), left=left, right=right)
        q.tanh(fx.view, fo.view)
        fo.assert_frame_untouched(("tanh", dt, rows, cols, left, right))


def test_elementwise_keeps_inside_rank3_views_with_gaps():
    g = H.rng(802)
    q = srt.current_queue()
    x = g.integers(-6, 7, (3, 17, 72)).astype(np.float32)
    y = g.integers(-6, 7, (3, 17, 72)).astype(np.float32)
    for left, right in [(8, 8), (1, 2)]:
        fx, fy = Framed(H.encode(x, H.BF16), left=left, right=right), Framed(H.encode(y, H.BF16), left=left, right=right)
        fo = Framed(np.zeros((3, 17, 72), np.uint16), left=left, right=right)
        q.add(fx.view, fy.view, fo.view)
        assert np.array_equal(fo.inside(), H.encode(x + y, H.BF16))
        fo.assert_frame_untouched(("add rank 3", left, right))


# ---- backward epilogue ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", [H.BF16, H.F32])
@pytest.mark.parametrize("no_alloc", [False, True])
def test_activation_backward_keeps_inside_its_views(dt, no_alloc):
    g = H.rng(803)
    q = srt.current_queue()
    for (rows, cols, left, right) in [(300, 520, 8, 8), (77, 1000, 8, 8), (45, 517, 3, 2), (600, 8, 8, 8)]:
        y = g.integers(-3, 4, (rows, cols)).astype(np.float32)
        dy = g.integers(-3, 4, (rows, cols)).astype(np.float32)
        fy, fdy = Framed(H.encode(y, dt), left=left, right=right), Framed(H.encode(dy, dt), left=left, right=right)
        fdx = Framed(H.encode(np.zeros((rows, cols), np.float32), dt), left=left, right=right)
        fdb = Framed(H.encode(np.zeros((1, cols), np.float32), dt), top=1, left=left, right=right)
        dbias = srt.Tensor(shape=[cols], order=fdb.view.order, _storage=fdb.view.storage, _offset=fdb.view.offset, _strides=[1])
        # (every tensor resident before the call: the mirror's staging must not be what allocates)
        for f in (fy, fdy, fdx, fdb):
            f.view.device_read(q)
        q.activation_backward(fy.view, fdy.view, srt.ActivationType.relu, 0.0, fdx.view, dbias, no_alloc=no_alloc)
        dx = dy * (y > 0)
        what = (dt, rows, cols, left, right, no_alloc)
        assert np.array_equal(fdx.inside()[0], H.encode(dx, dt).view(fdx.bits)), what
        assert np.array_equal(fdb.inside()[0, 0], H.encode(dx.sum(axis=0), dt).view(fdb.bits)), what
        fdx.assert_frame_untouched(what)
        fdb.assert_frame_untouched(what)
        fy.assert_unchanged(what)
        fdy.assert_unchanged(what)
