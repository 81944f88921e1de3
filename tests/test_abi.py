"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares,
descriptor marshalling, host-side shape logic.  No compute calls (no GPU here)."""
import ctypes
import os
import re

import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "srt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(srt[A-Z]\w*)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 28
    L = ctypes.CDLL(native.LIB_PATH)
    for n in names:
        assert hasattr(L, n), f"{n} declared in srt_hip.h but not exported"
    # and the binding table covers the header exactly
    assert sorted(native.SIGNATURES) == names


def test_status_strings_and_version():
    L = native.lib()
    assert L.srtGetVersion() >= 100
    assert L.srtGetStatusString(0) == b"srtSuccess"
    assert L.srtGetStatusString(801) == b"srtErrorNotSupported"
    assert L.srtGetStatusString(12345) == b"srtErrorUnknown"


def test_status_mapping_to_exceptions():
    native.check(0)
    with pytest.raises(srt.NotSupportedError):
        native.check(native.ERROR_NOT_SUPPORTED, "x")
    with pytest.raises(srt.SrtError) as e:
        native.check(native.ERROR_INVALID_VALUE, "x")
    assert not isinstance(e.value, srt.NotSupportedError)


def test_descriptor_marshalling():
    d, keep = native.make_descriptor(native.REAL16BF, (4, 6), (12, 2), native.ORDER_ROW)
    assert d.rank == 2 and d.count == 24 and d.spanCount == 3 * 12 + 5 * 2 + 1
    assert [d.shape[i] for i in range(2)] == [4, 6] and [d.strides[i] for i in range(2)] == [12, 2]
    assert [d.logicalStrides[i] for i in range(2)] == [6, 1]
    assert ctypes.sizeof(native.TensorDescriptor) == 56   # 3 x int32 + pad, 2 x size_t, 3 pointers


def test_descriptor_validation_without_gpu():
    # argument checks run before any device work, so they are observable on a CPU-only host
    L = native.lib()
    ad, k1 = native.make_descriptor(native.REAL32F, (3, 2), (2, 1), native.ORDER_ROW)
    bd, k2 = native.make_descriptor(native.REAL32F, (3, 4), (4, 1), native.ORDER_ROW)   # inner dims differ
    od, k3 = native.make_descriptor(native.REAL32F, (3, 4), (4, 1), native.ORDER_ROW)
    dummy = ctypes.c_void_p(256)
    assert L.srtMatmul(dummy, ctypes.byref(ad), 0, dummy, ctypes.byref(bd), 0, dummy, ctypes.byref(od), None) \
        == native.ERROR_INVALID_VALUE
    # double precision is not part of the path -> caller falls back
    a64, k4 = native.make_descriptor(native.REAL64F, (3, 2), (2, 1), native.ORDER_ROW)
    b64, k5 = native.make_descriptor(native.REAL64F, (2, 4), (4, 1), native.ORDER_ROW)
    o64, k6 = native.make_descriptor(native.REAL64F, (3, 4), (4, 1), native.ORDER_ROW)
    assert L.srtMatmul(dummy, ctypes.byref(a64), 0, dummy, ctypes.byref(b64), 0, dummy, ctypes.byref(o64), None) \
        == native.ERROR_NOT_SUPPORTED
    # tiled order -> not supported
    at, k7 = native.make_descriptor(native.REAL32F, (3, 2), (2, 1), 2)
    b2, k8 = native.make_descriptor(native.REAL32F, (2, 4), (4, 1), native.ORDER_ROW)
    assert L.srtMatmul(dummy, ctypes.byref(at), 0, dummy, ctypes.byref(b2), 0, dummy, ctypes.byref(od), None) \
        == native.ERROR_NOT_SUPPORTED
    # empty result: success, nothing launched
    ae, k9 = native.make_descriptor(native.REAL32F, (0, 2), (2, 1), native.ORDER_ROW)
    oe, k10 = native.make_descriptor(native.REAL32F, (0, 4), (4, 1), native.ORDER_ROW)
    assert L.srtMatmul(None, ctypes.byref(ae), 0, dummy, ctypes.byref(b2), 0, None, ctypes.byref(oe), None) == 0
    # null descriptor
    assert L.srtMatmul(dummy, None, 0, dummy, ctypes.byref(b2), 0, dummy, ctypes.byref(od), None) \
        == native.ERROR_INVALID_VALUE


def test_result_alias_rules_without_gpu():
    # The alias check runs on addresses and strides alone, before any device work: the refusals are observable
    # on a CPU-only host (the accepted cases go on to a launch and are tested on the GPU).
    L = native.lib()
    base = 1 << 20

    def call(a_off, a_shape, a_strides, o_off, o_shape, o_strides, b_shape=None):
        ad, k1 = native.make_descriptor(native.REAL32F, a_shape, a_strides, native.ORDER_ROW)
        kk = a_shape[-1]
        bs = b_shape or ((kk, o_shape[-1]) if len(a_shape) == 2 else (a_shape[0], kk, o_shape[-1]))
        bst = (bs[-1], 1) if len(bs) == 2 else (bs[-2] * bs[-1], bs[-1], 1)
        bd, k2 = native.make_descriptor(native.REAL32F, bs, bst, native.ORDER_ROW)
        od, k3 = native.make_descriptor(native.REAL32F, o_shape, o_strides, native.ORDER_ROW)
        return L.srtMatmul(ctypes.c_void_p(base + 4 * a_off), ctypes.byref(ad), 0, ctypes.c_void_p(1 << 30), ctypes.byref(bd), 0,
                           ctypes.c_void_p(base + 4 * o_off), ctypes.byref(od), None)

    # the same first element: provably aliased
    assert call(0, (32, 32), (64, 1), 0, (32, 32), (64, 1)) == native.ERROR_INVALID_VALUE
    # overlapping row blocks of one 64-wide buffer, same columns: provably aliased
    assert call(0, (32, 32), (64, 1), 16 * 64, (32, 32), (64, 1)) == native.ERROR_INVALID_VALUE
    # row blocks that overlap with column ranges that meet in part: provably aliased too
    assert call(0, (32, 32), (64, 1), 16 * 64 + 16, (32, 32), (64, 1)) == native.ERROR_INVALID_VALUE
    # spans overlap, pitches differ: the check cannot tell -> the caller's fallback
    assert call(0, (32, 32), (64, 1), 40, (32, 32), (48, 1)) == native.ERROR_NOT_SUPPORTED
    # a transposed view covers the same elements as the block it transposes: provably aliased with a result 8 columns along
    assert call(0, (32, 32), (1, 64), 8, (32, 32), (64, 1)) == native.ERROR_INVALID_VALUE
    # rows of 32 under a pitch of 96 against rows under a pitch of 64, 8 elements in: apart or not, no pitch shows it
    assert call(0, (32, 32), (96, 1), 8, (32, 32), (64, 1)) == native.ERROR_NOT_SUPPORTED


def test_result_alias_rule_never_accepts_views_that_share_an_element():
    """Random small views (all strides, pitches and offsets inside one buffer), checked against the element sets written
    out: whenever the result shares an element with an operand the call must be refused (either status); the proof of
    disjointness may fail to find what is true, never claim what is false.  Accepted calls go on to a launch, so this runs
    only where there is no device to launch on (placeholder pointers)."""
    L = native.lib()
    count = ctypes.c_int32(0)
    if L.srtGetDeviceCount(ctypes.byref(count)) == 0 and count.value > 0:
        pytest.skip("placeholder pointers: only on a host without a device")
    g = np.random.Generator(np.random.Philox(1234))
    refusals = (native.ERROR_INVALID_VALUE, native.ERROR_NOT_SUPPORTED)

    # the verdict depends on where the views lie relative to one another, not on where the buffer lies: interleaved
    # batches and column slices are told apart at any base address (a pitch of 3072 bytes against bases 1 KiB apart)
    for shift in (0, 4, 1024, 2048, 1536, 3068, 12345 * 4):
        base = (1 << 22) + shift
        ad, k1 = native.make_descriptor(native.REAL32F, (3, 16, 24), (768, 24, 1), native.ORDER_ROW)
        bd, k2 = native.make_descriptor(native.REAL32F, (3, 24, 24), (576, 24, 1), native.ORDER_ROW)
        st = L.srtMatmul(ctypes.c_void_p(base), ctypes.byref(ad), 0, ctypes.c_void_p(1 << 30), ctypes.byref(bd), 0,
                         ctypes.c_void_p(base + 4 * 384), ctypes.byref(ad), None)
        assert st not in refusals, shift
        ad, k1 = native.make_descriptor(native.REAL32F, (48, 32), (96, 1), native.ORDER_ROW)
        bd, k2 = native.make_descriptor(native.REAL32F, (32, 32), (32, 1), native.ORDER_ROW)
        st = L.srtMatmul(ctypes.c_void_p(base), ctypes.byref(ad), 0, ctypes.c_void_p(1 << 30), ctypes.byref(bd), 0,
                         ctypes.c_void_p(base + 4 * 64), ctypes.byref(ad), None)
        assert st not in refusals, shift
        # ... and the same views one row further along than a whole pitch apart still share their elements
        st = L.srtMatmul(ctypes.c_void_p(base), ctypes.byref(ad), 0, ctypes.c_void_p(1 << 30), ctypes.byref(bd), 0,
                         ctypes.c_void_p(base + 4 * (96 + 16)), ctypes.byref(ad), None)
        assert st == native.ERROR_INVALID_VALUE, shift

    def view(rows, cols):
        kind = int(g.integers(0, 4))
        if kind == 0:       # dense rows under a pitch
            pitch = cols + int(g.integers(0, 12))
            st = (pitch, 1)
        elif kind == 1:     # transposed: columns under a pitch
            pitch = rows + int(g.integers(0, 12))
            st = (1, pitch)
        elif kind == 2:     # every other element of a row
            pitch = 2 * cols + int(g.integers(0, 8))
            st = (pitch, 2)
        else:               # arbitrary
            st = (int(g.integers(1, 40)), int(g.integers(1, 40)))
        return int(g.integers(0, 64)), st

    def elements(off, shape, st):
        return {off + i * st[0] + j * st[1] for i in range(shape[0]) for j in range(shape[1])}

    refused = accepted = overlapping = 0
    for _ in range(3000):
        M, N, K = int(g.integers(1, 7)), int(g.integers(1, 7)), int(g.integers(1, 7))
        a_off, a_st = view(M, K)
        o_off, o_st = view(M, N)
        ad, k1 = native.make_descriptor(native.REAL32F, (M, K), a_st, native.ORDER_ROW)
        bd, k2 = native.make_descriptor(native.REAL32F, (K, N), (N, 1), native.ORDER_ROW)
        od, k3 = native.make_descriptor(native.REAL32F, (M, N), o_st, native.ORDER_ROW)
        base = (1 << 22) + 4 * int(g.integers(0, 4096))
        st = L.srtMatmul(ctypes.c_void_p(base + 4 * a_off), ctypes.byref(ad), 0, ctypes.c_void_p(1 << 30), ctypes.byref(bd), 0,
                         ctypes.c_void_p(base + 4 * o_off), ctypes.byref(od), None)
        shares = bool(elements(a_off, (M, K), a_st) & elements(o_off, (M, N), o_st))
        overlapping += shares
        if st in refusals:
            refused += 1
        else:
            accepted += 1
            assert not shares, (M, N, K, a_off, a_st, o_off, o_st)
    # the draw exercises both answers and both truths
    assert overlapping > 300 and accepted > 300 and refused > 300, (overlapping, accepted, refused)


def test_elementwise_and_backward_validation_without_gpu():
    L = native.lib()
    dummy = ctypes.c_void_p(256)
    ad, k1 = native.make_descriptor(native.REAL32F, (4, 8), (8, 1), native.ORDER_ROW)
    bd, k2 = native.make_descriptor(native.REAL32F, (4, 9), (9, 1), native.ORDER_ROW)
    d64, k3 = native.make_descriptor(native.REAL64F, (4, 8), (8, 1), native.ORDER_ROW)
    vec, k4 = native.make_descriptor(native.REAL32F, (8,), (1,), native.ORDER_ROW)
    for name in ("srtAdd", "srtSub", "srtMul", "srtDiv", "srtMax", "srtMin"):
        f = getattr(L, name)
        assert f(dummy, ctypes.byref(ad), dummy, ctypes.byref(bd), dummy, ctypes.byref(ad), None) \
            == native.ERROR_INVALID_VALUE                       # shapes differ
        assert f(dummy, ctypes.byref(d64), dummy, ctypes.byref(d64), dummy, ctypes.byref(d64), None) \
            == native.ERROR_NOT_SUPPORTED                       # element type: caller's CPU fallback
        assert f(dummy, None, dummy, ctypes.byref(ad), dummy, ctypes.byref(ad), None) == native.ERROR_INVALID_VALUE
        assert getattr(L, name + "TE")(dummy, ctypes.byref(ad), None, dummy, ctypes.byref(ad), None) \
            == native.ERROR_INVALID_VALUE                       # no element
    for name in ("srtNeg", "srtExp", "srtSigmoid", "srtTanh"):
        assert getattr(L, name)(dummy, ctypes.byref(ad), dummy, ctypes.byref(d64), None) == native.ERROR_NOT_SUPPORTED
        assert getattr(L, name)(dummy, ctypes.byref(ad), dummy, ctypes.byref(vec), None) == native.ERROR_INVALID_VALUE
    assert L.srtCopy(dummy, ctypes.byref(d64), dummy, ctypes.byref(ad), None) == native.ERROR_NOT_SUPPORTED
    assert L.srtAddFlat(native.REAL64F, dummy, dummy, dummy, 16, None) == native.ERROR_NOT_SUPPORTED
    assert L.srtAddFlat(native.REAL32F, dummy, dummy, dummy, 0, None) == native.SUCCESS
    assert L.srtCopyFlat(native.REAL32F, None, native.REAL16BF, dummy, 16, None) == native.ERROR_INVALID_VALUE
    assert L.srtFillFlat(native.REAL32F, dummy, None, 16, None) == native.ERROR_INVALID_VALUE
    # empty tensors: success before any pointer is looked at
    e, k5 = native.make_descriptor(native.REAL32F, (0, 8), (8, 1), native.ORDER_ROW)
    assert L.srtAdd(None, ctypes.byref(e), None, ctypes.byref(e), None, ctypes.byref(e), None) == native.SUCCESS
    # backward: extents, activation code, element type, rank
    f = L.srtActivationBackwardBias
    assert f(dummy, ctypes.byref(ad), dummy, ctypes.byref(bd), 1, 0.0, dummy, ctypes.byref(ad), None, None, None) \
        == native.ERROR_INVALID_VALUE
    assert f(dummy, ctypes.byref(ad), dummy, ctypes.byref(ad), 6, 0.0, dummy, ctypes.byref(ad), None, None, None) \
        == native.ERROR_INVALID_VALUE
    assert f(dummy, ctypes.byref(d64), dummy, ctypes.byref(d64), 1, 0.0, dummy, ctypes.byref(d64), None, None, None) \
        == native.ERROR_NOT_SUPPORTED
    assert f(dummy, ctypes.byref(vec), dummy, ctypes.byref(vec), 1, 0.0, dummy, ctypes.byref(vec), None, None, None) \
        == native.ERROR_NOT_SUPPORTED
    bad_bias, k6 = native.make_descriptor(native.REAL32F, (9,), (1,), native.ORDER_ROW)
    assert f(dummy, ctypes.byref(ad), dummy, ctypes.byref(ad), 1, 0.0, dummy, ctypes.byref(ad), dummy,
             ctypes.byref(bad_bias), None) == native.ERROR_INVALID_VALUE


def test_repeating_views_and_gradient_table_shapes():
    b = srt.Tensor(np.arange(4, dtype=np.float32))
    r = srt.Tensor.repeating(b, (3, 4))
    assert r.shape == (3, 4) and r.strides == (0, 1)
    c = srt.Tensor(np.zeros((3, 1), np.float32))
    assert srt.Tensor.repeating(c, (3, 5)).strides == (1, 0)
    with pytest.raises(ValueError):
        srt.Tensor.repeating(b, (3, 5))
    assert srt.Tensor(np.zeros((2, 3), np.float32)).is_contiguous
    assert not srt.Tensor(np.zeros((4, 6), np.float32))[:, 1:4].is_contiguous
    assert srt.Tensor(np.zeros(2, np.uint16)).element_storage(1.0)[0] == 0x3F80
    assert srt.Tensor(np.zeros(2, np.uint16)).element_storage(float("nan"))[0] == 0x7FFF


def test_plan_cache_file_round_trip_and_rejects_malformed_files(tmp_path):
    """Save / Load of the plan cache are host-only: a plan written by hand is loaded, counted, saved
    back identically; unknown plan names, short lines and missing files change nothing."""
    srt.PlanCache.clear()
    assert srt.PlanCache.count() == 0
    good = tmp_path / "plans.txt"
    good.write_text("# comment\n14 2048 2048 2048 1 89 10 mfma_128x128\n0 512 512 512 1 89 10 f32_mfma_splitk\n")
    srt.PlanCache.load(good)
    assert srt.PlanCache.count() == 2
    out = tmp_path / "saved.txt"
    srt.PlanCache.save(out)
    lines = [ln for ln in out.read_text().splitlines() if not ln.startswith("#")]
    assert sorted(lines) == sorted(["14 2048 2048 2048 1 89 10 mfma_128x128", "0 512 512 512 1 89 10 f32_mfma_splitk"])
    for text in ("14 2048 2048 2048 1 89 10 no_such_plan\n", "14 2048 2048\n", "14 64 64 64 1 89 10 generic\nx y z\n"):
        bad = tmp_path / "bad.txt"
        bad.write_text(text)
        with pytest.raises(srt.SrtError):
            srt.PlanCache.load(bad)
        assert srt.PlanCache.count() == 2                       # all or nothing
    with pytest.raises(srt.SrtError):
        srt.PlanCache.load(tmp_path / "missing.txt")
    # a loaded plan steers the (GPU-free) kernel query for that key; clearing restores the heuristic
    ad, k1 = native.make_descriptor(native.REAL16BF, (2048, 2048), (2048, 1), native.ORDER_ROW)
    buf = ctypes.create_string_buffer(64)
    dummy = ctypes.c_void_p(4096)
    L = native.lib()
    assert L.srtMatmulQueryKernel(ctypes.byref(ad), 0, ctypes.byref(ad), 0, ctypes.byref(ad), dummy, dummy, dummy,
                                  buf, 64) == 0
    assert buf.value == b"mfma_128x128"
    srt.PlanCache.clear()
    assert L.srtMatmulQueryKernel(ctypes.byref(ad), 0, ctypes.byref(ad), 0, ctypes.byref(ad), dummy, dummy, dummy,
                                  buf, 64) == 0
    assert buf.value == b"mfma_128x128_m16_k128"
    assert L.srtPlanCacheCount(None) == native.ERROR_INVALID_VALUE
    assert L.srtPlanCacheLoad(None) == native.ERROR_INVALID_VALUE


def test_kernel_selection_is_queryable_without_gpu():
    L = native.lib()

    def query(dt, M, N, K, ta=False, tb=False, align=256):
        ashape = (K, M) if ta else (M, K)
        bshape = (N, K) if tb else (K, N)
        ad, k1 = native.make_descriptor(dt, ashape, (ashape[1], 1), native.ORDER_ROW)
        bd, k2 = native.make_descriptor(dt, bshape, (bshape[1], 1), native.ORDER_ROW)
        od, k3 = native.make_descriptor(dt, (M, N), (N, 1), native.ORDER_ROW)
        buf = ctypes.create_string_buffer(64)
        p = ctypes.c_void_p(align)
        st = L.srtMatmulQueryKernel(ctypes.byref(ad), int(ta), ctypes.byref(bd), int(tb), ctypes.byref(od),
                                    p, p, p, buf, 64)
        assert st == 0
        return buf.value.decode()

    # a full device: the 16x16x32 kernel with 64-deep staging units, in every layout
    assert query(native.REAL16BF, 8192, 8192, 8192) == "mfma_256x256_m16_k64"
    assert query(native.REAL16BF, 8192, 8192, 8192, ta=True) == "mfma_256x256_m16_k64"
    assert query(native.REAL16BF, 4096, 11008, 4096) == "mfma_256x256_m16_k64"
    assert query(native.REAL16BF, 8192, 8192, 8192, tb=True) == "mfma_256x256_m16_k64"
    # short k loops: the same (two k-contiguous operands used to take the 32x32x16 kernel with 64-deep stages)
    assert query(native.REAL16BF, 4096, 4096, 1024) == "mfma_256x256_m16_k64"
    assert query(native.REAL16BF, 4096, 4096, 1024, tb=True) == "mfma_256x256_m16_k64"
    # few tiles and a long k loop: K split over the idle compute units -- when that buys more than the
    # half-height tiles a k-contiguous A allows
    assert query(native.REAL16BF, 128, 2048, 4096) == "mfma_256x256_splitk"           # eight half tiles in eight parts (18.5 us against 25 in quarter tiles)
    assert query(native.REAL16BF, 128, 2048, 4096, tb=True) == "mfma_256x256_splitk"
    assert query(native.REAL16BF, 256, 1024, 8192) == "mfma_256x256_splitk"           # four whole tiles in sixteen parts
    # ... unless one round of 128 x 128 quarter tiles holds the problem and the k loop is short enough for them (K <= 2048: always;
    # 4096: from 48 tiles; beyond: from K / 73 tiles)
    assert query(native.REAL16BF, 512, 4096, 4096) == "mfma_128x128_m16_k128"         # 128 quarter tiles (25.5 us against 38 in parts)
    assert query(native.REAL16BF, 512, 4096, 4096, tb=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 512, 1536, 4096) == "mfma_128x128_m16_k128"         # 48
    assert query(native.REAL16BF, 256, 2048, 4096) == "mfma_256x256_splitk"           # 32: a tie with eight parts (24.4 us against 24.1-25.9)
    assert query(native.REAL16BF, 384, 1536, 4096) == "mfma_128x128_m16_k128"         # 36 (25.0-25.2 against 24.9-26.0)
    assert query(native.REAL16BF, 8, 1728, 3200, ta=True, tb=True) == "mfma_128x128_m16_k128"   # K = 3200 only goes in four parts of 800: 20.0 us against 24.5
    assert query(native.REAL16BF, 476, 1936, 8448) == "mfma_256x256_splitk"           # eight parts of 1056 against a k loop of 8448: 35.5 us against 45.2
    assert query(native.REAL16BF, 512, 2048, 8192) == "mfma_256x256_splitk"           # 64 at K = 8192: parts
    assert query(native.REAL16BF, 1024, 4096, 4096) == "mfma_128x128_m16_k128"        # 256 quarter tiles (31.8 us against 42 shared)
    # 64 to 160 whole tiles beyond one round of quarter tiles: the tail-sharing form of the 64-deep kernel (every tile cut
    # along k into two or three parts), unless half-height tiles fill one round as well
    assert query(native.REAL16BF, 2048, 4096, 4096, tb=True) == "mfma_128x256_m16_k64"
    assert query(native.REAL16BF, 2048, 4096, 4096) == "mfma_128x256_m16_k64"
    assert query(native.REAL16BF, 2048, 4096, 8192) == "mfma_256x256_m16_k64_tail"
    assert query(native.REAL16BF, 4096, 10240, 4096) == "mfma_256x256_m16_k64"        # after whole rounds it buys nothing
    assert query(native.REAL16BF, 2048, 2048, 8192) == "mfma_128x128_m16_k128"        # 256 quarter tiles, K = 8192 (59 us against 63-66 shared)
    assert query(native.REAL16BF, 1024, 2048, 8192) == "mfma_128x128_m16_k128"        # 128 of them
    assert query(native.REAL16BF, 256, 8192, 8192, ta=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 256, 4096, 8192, ta=True) == "mfma_256x256_splitk"      # 64: parts
    assert query(native.REAL16BF, 1024, 2048, 2048, ta=True) == "mfma_128x128_m16_k128"   # any layout
    assert query(native.REAL16BF, 1024, 2048, 1024, ta=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 1024, 1024, 1024, ta=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 1024, 8192, 2048, ta=True) == "mfma_256x128_m16_k64"    # 512 quarter tiles: A not k-contiguous, one round of its 256 x 128 half tiles
    assert query(native.REAL16BF, 1024, 8192, 1920, ta=True) == "mfma_256x128_m16_k64"    # (so too where K is no whole number of 128-deep units)
    assert query(native.REAL16BF, 1024, 2048, 1984, ta=True) == "mfma_256x128_m16_k64"
    # mid-size problems: the 256 x 256 kernels from 24 tiles up (96 when both operands are k-contiguous),
    # 64 x 64 tiles below, so that every CU gets a workgroup
    assert query(native.REAL16BF, 3072, 3072, 3072) == "mfma_256x256_m16_k64"             # 144 tiles, long k loop
    assert query(native.REAL16BF, 3072, 3072, 1024) == "mfma_256x256_m16_k64"             # and a short one
    # a k-contiguous A and at most one round of 128 x 256 tiles: the half-height form of the 16x16x32 kernel -- beyond one
    # round of quarter tiles, or where K is no whole number of their 128-deep units
    assert query(native.REAL16BF, 2048, 2048, 2048) == "mfma_128x128_m16_k128"            # 256 quarter tiles (18.5 us against 24-26 in half tiles)
    assert query(native.REAL16BF, 2048, 2048, 2048, tb=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 2048, 2048, 1984) == "mfma_128x256_m16_k64"             # 128 half tiles
    assert query(native.REAL16BF, 2048, 2048, 1984, tb=True) == "mfma_128x256_m16_k64"
    assert query(native.REAL16BF, 2048, 4096, 2048) == "mfma_128x256_m16_k64"             # 256 half tiles
    assert query(native.REAL16BF, 2048, 2048, 2048, ta=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 2048, 2048, 1984, ta=True) == "mfma_256x128_m16_k64"    # A not k-contiguous: its half tile is 256 x 128
    assert query(native.REAL16BF, 2048, 2048, 1024, ta=True) == "mfma_128x128_m16_k128"
    # 258 whole tiles: a whole round, and the two left over cut along k in three parts each
    assert query(native.REAL16BF, 1536, 11008, 4096) == "mfma_256x256_m16_k64_tail"
    assert query(native.REAL16BF, 1536, 11008, 4096, tb=True) == "mfma_256x256_m16_k64_tail"
    assert query(native.REAL16BF, 1536, 11008, 2048) == "mfma_256x256_m16_k64"        # (not for a k loop this short)
    assert query(native.REAL16BF, 1536, 4096, 11008, tb=True) == "mfma_256x256_m16_k64_tail"   # 96 tiles, two parts each
    assert query(native.REAL16BF, 256, 1024, 1024) == "mfma_128x128_m16_k128"             # 16 quarter tiles
    assert query(native.REAL16BF, 256, 1024, 960) == "mfma_128x256_m16_k64"               # 8 half tiles
    assert query(native.REAL16BF, 1024, 1024, 2048, tb=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 1024, 1024, 1984, tb=True) == "mfma_64x64"          # 32 half tiles, both k-contiguous
    assert query(native.REAL16BF, 512, 4096, 2048) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 512, 4096, 1984) == "mfma_128x256_m16_k64"              # K too short to split
    assert query(native.REAL16BF, 512, 4096, 256) == "mfma_128x128_m16_k128"              # short k loops too (two 128-deep units)
    assert query(native.REAL16BF, 512, 4096, 192) == "mfma_128x256_m16"                   # (8.4 us against 10.0 in whole tiles)
    assert query(native.REAL16F, 256, 256, 256, tb=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16F, 256, 256, 192, tb=True) == "mfma_64x64"
    assert query(native.REAL16BF, 1, 14336, 4096, tb=True) == "skinny"
    assert query(native.REAL16BF, 32, 14336, 4096, tb=True) == "skinny"
    # 33..64 rows: the streaming kernel when its workgroups make one round that fills the device
    assert query(native.REAL16BF, 64, 14336, 4096, tb=True) == "skinny"               # 224 workgroups of 64 weight rows
    assert query(native.REAL16BF, 64, 4096, 4096, tb=True) == "skinny"                # 128 of 32, short enough k loop
    assert query(native.REAL16BF, 64, 4096, 14336, tb=True) == "mfma_256x256_splitk"  # few workgroups, long k loop
    assert query(native.REAL16BF, 64, 11008, 4096, tb=True) == "mfma_256x256_splitk"  # 344 workgroups: not one round
    assert query(native.REAL16BF, 65, 14336, 4096, tb=True) == "mfma_128x128_m16_k128"  # 112 quarter tiles, half padding
    assert query(native.REAL16BF, 65, 14336, 4032, tb=True) == "mfma_256x256_splitk"
    # fp32, up to 32 rows against a k-contiguous weight: the streaming kernel too (four k values per 16-byte chunk)
    assert query(native.REAL32F, 1, 14336, 4096, tb=True) == "skinny"
    assert query(native.REAL32F, 32, 256, 1024, tb=True) == "skinny"
    assert query(native.REAL32F, 32, 14336, 4098, tb=True) == "f32_mfma"              # K not in whole 16-byte chunks
    assert query(native.REAL32F, 33, 14336, 4096, tb=True) == "f32_mfma"
    assert query(native.REAL32F, 8, 14336, 4096) == "skinny"                          # an n-contiguous weight likewise
    assert query(native.REAL32F, 8, 14338, 4096) == "f32_mfma"                        # its rows not in whole chunks
    assert query(native.REAL32F, 8, 14336, 4096, ta=True) == "f32_mfma"               # x must be k-contiguous
    # x . W with an n-contiguous W: the streaming kernel within one round of 64-column workgroups and a short k loop
    assert query(native.REAL16BF, 8, 14336, 4096) == "skinny"
    assert query(native.REAL16BF, 32, 4096, 2048) == "skinny"
    assert query(native.REAL16BF, 32, 4096, 4096) == "mfma_256x256_splitk"            # 64 workgroups, 17..32 rows
    assert query(native.REAL16BF, 8, 4096, 8192) == "mfma_256x256_splitk"             # long k loop
    assert query(native.REAL16BF, 8, 28672, 1024) == "mfma_128x256_m16_k64"               # 448 workgroups: not one round
    assert query(native.REAL16BF, 64, 14336, 4096) == "mfma_128x128_m16_k128"         # 64 rows against an n-contiguous W: quarter tiles from 48 up
    assert query(native.REAL16BF, 64, 11008, 4096) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 64, 14336, 4032) == "skinny"
    # what sweeps against every pinned plan found (the measured pairs stand next to the rules in csrc/gemm_mfma.hip)
    assert query(native.REAL16BF, 24, 96, 10320) == "skinny"                          # K / 2 is not a whole number of stages: no split-K
    assert query(native.REAL16BF, 8, 1288, 10432) == "skinny"                         # only two parts possible
    assert query(native.REAL16BF, 8, 88, 2576, ta=True) == "mfma_256x256_m16"           # one whole tile beats 64 x 64 tiles on an m-contiguous A
    assert query(native.REAL16BF, 4826, 12408, 7056, tb=True) == "mfma_256x256_k64"   # k extent not a whole number of 32-deep stages
    assert query(native.REAL16BF, 192, 12568, 3264, ta=True, tb=True) == "mfma_256x128_m16_k64"   # K only halves: one round of half tiles beats two parts
    assert query(native.REAL16BF, 664, 7536, 352, tb=True) == "mfma_128x256_m16"      # 13 % padding rows are fine for half tiles
    assert query(native.REAL16BF, 169, 9824, 504, tb=True) == "mfma_64x64"            # a second row of half tiles that is mostly padding is not
    assert query(native.REAL16BF, 512, 512, 1024, ta=True) == "mfma_128x128_m16_k128"  # sixteen quarter tiles (9.9 us against 15.8 in half tiles)
    assert query(native.REAL16BF, 8, 14336, 4096, ta=True, tb=True) == "mfma_128x128_m16_k128"   # a handful of rows of an m-contiguous A: no streaming kernel, 112 quarter tiles beat the parts
    assert query(native.REAL16BF, 32, 4096, 2048, ta=True) == "mfma_128x128_m16_k128"
    assert query(native.REAL16BF, 32, 4096, 4096, ta=True) == "mfma_256x256_splitk"              # 32 tiles at K = 4096: parts
    assert query(native.REAL16BF, 512, 512, 960, ta=True) == "mfma_256x128_m16_k64"    # eight half tiles, neither operand k-contiguous: ahead of split-K
    # batches (no split-K pass)
    def query_batched(dt, B, M, N, K, ta=False, tb=False):
        ashape = (B, K, M) if ta else (B, M, K)
        bshape = (B, N, K) if tb else (B, K, N)
        ad, k1 = native.make_descriptor(dt, ashape, (ashape[1] * ashape[2], ashape[2], 1), native.ORDER_ROW)
        bd, k2 = native.make_descriptor(dt, bshape, (bshape[1] * bshape[2], bshape[2], 1), native.ORDER_ROW)
        od, k3 = native.make_descriptor(dt, (B, M, N), (M * N, N, 1), native.ORDER_ROW)
        buf = ctypes.create_string_buffer(64)
        p = ctypes.c_void_p(256)
        assert L.srtMatmulQueryKernel(ctypes.byref(ad), int(ta), ctypes.byref(bd), int(tb), ctypes.byref(od), p, p, p, buf, 64) == 0
        return buf.value.decode()
    assert query_batched(native.REAL16F, 32, 256, 256, 256, tb=True) == "mfma_128x128_m16_k128"        # benchmark config 2: launch-sized, 128 quarter tiles (6.4 us against 7.0-7.2 in 64 x 64 tiles)
    assert query_batched(native.REAL16F, 32, 256, 256, 192, tb=True) == "mfma_64x64"                   # every CU a workgroup
    assert query_batched(native.REAL16BF, 16, 384, 384, 1024, tb=True) == "mfma_128x128_m16_k128"      # 144 quarter tiles of a batch (15.0 us against 16.1 in half tiles)
    assert query_batched(native.REAL16BF, 16, 384, 384, 960, tb=True) == "mfma_128x256_m16_k64"        # 96 half tiles of a batch, 64 deep
    assert query_batched(native.REAL16BF, 16, 64, 512, 1024, ta=True) == "mfma_128x128_m16_k128"       # 64 quarter tiles, half padding
    assert query_batched(native.REAL16BF, 16, 64, 512, 960, ta=True) == "mfma_256x128_m16_k64"         # 64 tiles of 256 x 128, A not k-contiguous
    assert query_batched(native.REAL16BF, 4, 256, 256, 4096, ta=True) == "mfma_128x128_m16_k128"       # 16 quarter tiles (24 us against 40 shared: a batch has no split-K)
    assert query_batched(native.REAL16BF, 16, 256, 256, 2048, ta=True, tb=True) == "mfma_128x128_m16_k128"
    assert query_batched(native.REAL16BF, 4, 128, 128, 4096, tb=True) == "mfma_128x128_m16_k128"
    assert query_batched(native.REAL16BF, 4, 128, 128, 4032, tb=True) == "mfma_64x64"                  # mostly padding, both k-contiguous
    assert query_batched(native.REAL16BF, 16, 512, 512, 4096) == "mfma_256x256_m16_k64_tail"           # 256 quarter tiles of small problems: operand traffic
    assert query_batched(native.REAL16BF, 64, 256, 256, 1024, tb=True) == "mfma_128x256_m16_k64"           # 128 half tiles in one round
    assert query_batched(native.REAL16BF, 64, 256, 1024, 256, tb=True) == "mfma_256x256_m16_k64"       # 512 half tiles: whole tiles
    assert query_batched(native.REAL16BF, 64, 384, 384, 4096, tb=True) == "mfma_256x256_k64"           # a last row of tiles half padding
    assert query_batched(native.REAL16BF, 28, 8, 88, 7680) == "skinny"                                 # ahead of sharing padded tiles
    assert query_batched(native.REAL16BF, 41, 1480, 72, 1248, tb=True) == "mfma_256x256_k64"           # a device's worth of padded whole tiles
    assert query_batched(native.REAL16BF, 36, 8, 768, 328, tb=True) == "mfma_64x64"                    # 864 streaming workgroups: not worth it
    # 16-bit operands that miss the 16-byte rules: the matrix-core kernel with element-wise staging
    assert query(native.REAL16BF, 33, 33, 33) == "mfma_64x64_any"
    assert query(native.REAL16BF, 64, 64, 64, align=2) == "mfma_64x64_any"            # misaligned view
    assert query(native.REAL16F, 2048, 50257, 768) == "mfma_128x128_any"              # odd row pitch of B and C
    assert query(native.REAL32F, 512, 512, 512) in ("generic", "f32_mfma")
    # operands of 1 Gi elements or more: halves of M (N for a k-contiguous B, the batch first) that the
    # 256 x 256 kernels' 32-bit offsets reach; a k walk out of reach keeps the small tiles
    assert query(native.REAL16BF, 32768, 32768, 8192) == "mfma_256x256_m16_k64/pieces"           # C alone is 1 Gi
    assert query(native.REAL16BF, 262144, 8192, 8192) == "mfma_256x256_m16_k64/pieces"           # A and C
    assert query(native.REAL16BF, 8192, 262144, 8192, tb=True) == "mfma_256x256_m16_k64/pieces"  # B [N, K] and C
    assert query(native.REAL16BF, 8192, 8192, 262144, ta=True) == "mfma_128x128"             # k walk of A and B
    assert query(native.REAL16BF, 32768, 32512, 8192) == "mfma_256x256_m16_k64"                  # just within reach
    assert query(native.REAL16BF, 8, 65664, 32768, tb=True) == "skinny/pieces"


def test_kernel_selection_answers_for_any_problem():
    """Random shapes, types, layouts, pitches, batches and alignments (zero extents included): the selection logic
    answers every one with success and a known plan name.  (Run against the host-sanitizer build of the library, this is
    also the fuzz of its arithmetic: `make -C swiftrt_amd/csrc SANITIZE=1`, SWIFTRT_HIP_LIBRARY.)"""
    L = native.lib()
    g = np.random.default_rng(123)
    buf = ctypes.create_string_buffer(64)
    known = {"empty", "generic", "skinny", "f32_mfma", "mfma_256x256", "mfma_128x128", "mfma_64x64", "mfma_256x256_k64",
             "mfma_256x256_m16", "mfma_256x256_splitk", "mfma_128x256_m16", "mfma_128x128_any", "mfma_64x64_any",
             "mfma_256x256_m16_k64", "mfma_256x256_m16_k64_tail", "mfma_256x256_m16_k64_split", "mfma_128x256_m16_k64", "mfma_256x128_m16_k64", "mfma_128x128_m16_k128"}

    def logu(lo, hi):
        return int(np.exp(g.uniform(np.log(lo), np.log(hi))))

    seen = set()
    for _ in range(4000):
        dt = [native.REAL16BF, native.REAL16F, native.REAL32F][int(g.integers(0, 3))]
        batch = 1 if g.random() < 0.7 else logu(1, 300)
        M, N, K = logu(1, 20000), logu(1, 40000), logu(1, 40000)
        if g.random() < 0.6:
            M, N, K = max(8, M // 8 * 8), max(8, N // 8 * 8), max(8, K // 8 * 8)
        if g.random() < 0.02:
            M = 0
        if g.random() < 0.02:
            K = 0
        ta, tb = int(g.integers(0, 2)), int(g.integers(0, 2))
        pa, pb, pc = [int(g.integers(0, 3)) * 8 if g.random() < 0.2 else 0 for _ in range(3)]
        ash = (K, M) if ta else (M, K)
        bsh = (N, K) if tb else (K, N)
        if batch > 1:
            ad = native.make_descriptor(dt, (batch,) + ash, (ash[0] * (ash[1] + pa), ash[1] + pa, 1), native.ORDER_ROW)
            bd = native.make_descriptor(dt, (batch,) + bsh, (bsh[0] * (bsh[1] + pb), bsh[1] + pb, 1), native.ORDER_ROW)
            od = native.make_descriptor(dt, (batch, M, N), (M * (N + pc), N + pc, 1), native.ORDER_ROW)
        else:
            ad = native.make_descriptor(dt, ash, (ash[1] + pa, 1), native.ORDER_ROW)
            bd = native.make_descriptor(dt, bsh, (bsh[1] + pb, 1), native.ORDER_ROW)
            od = native.make_descriptor(dt, (M, N), (N + pc, 1), native.ORDER_ROW)
        p = ctypes.c_void_p(256 if g.random() < 0.9 else int(g.integers(1, 16)) * 2)
        st = L.srtMatmulQueryKernel(ctypes.byref(ad[0]), ta, ctypes.byref(bd[0]), tb, ctypes.byref(od[0]), p, p, p, buf, 64)
        assert st == 0, (dt, batch, M, N, K, ta, tb)
        name = buf.value.decode()
        assert name.split("/")[0] in known and name.split("/")[-1] in known | {"pieces"}, name
        seen.add(name.split("/")[0])
    assert {"skinny", "mfma_64x64", "mfma_256x256_m16", "mfma_128x256_m16", "f32_mfma"} <= seen


def test_tensor_layout_and_views():
    t = srt.Tensor(np.arange(12, dtype=np.float32).reshape(3, 4))
    assert t.shape == (3, 4) and t.strides == (4, 1)
    assert t.t.shape == (4, 3) and t.t.strides == (1, 4)          # .t swaps extents and strides, zero copy
    assert np.array_equal(t.t.array(), np.arange(12, dtype=np.float32).reshape(3, 4).T)
    v = t[1:3, 1:4:2]
    assert v.shape == (2, 2) and v.strides == (4, 2) and v.offset == 5
    assert np.array_equal(v.array(), [[5, 7], [9, 11]])
    c = srt.Tensor(np.arange(6, dtype=np.float32).reshape(3, 2), order=srt.Order.col)
    assert c.strides == (1, 3)
    assert np.array_equal(c.array(), np.arange(6, dtype=np.float32).reshape(3, 2))
    t3 = srt.Tensor(np.zeros((2, 3, 4), np.float16))
    assert t3.t.shape == (2, 4, 3) and t3.t.strides == (12, 1, 4)  # only the last two dims swap


def test_matmul_shape_rules_raise_before_any_native_call():
    a = srt.Tensor(np.zeros((3, 2), np.float32))
    b = srt.Tensor(np.zeros((3, 4), np.float32))
    with pytest.raises(ValueError):
        srt.matmul(a, b)
    with pytest.raises(ValueError):
        srt.Dense(srt.Tensor(np.zeros((2, 4), np.float32)), bias=srt.Tensor(np.zeros(3, np.float32)))


def test_activation_enum_matches_reference_case_order():
    assert [a.name for a in srt.ActivationType] == ["sigmoid", "relu", "tanh", "clippedRelu", "elu", "identity"]
    assert [int(a) for a in srt.ActivationType] == list(range(6))


def test_bf16_fast_encoder_matches_oracle_codec():
    from oracle import srt_oracle as ora
    from tests import helpers
    r = np.random.default_rng(0)
    x = np.concatenate([r.standard_normal(100000).astype(np.float32),
                        np.array([0, -0.0, np.inf, -np.inf, np.nan, 1 + 2 ** -8, 1 + 3 * 2 ** -8, 3.4e38], np.float32)])
    assert np.array_equal(helpers.bf16_encode_fast(x), ora.encode(x, ora.BF16))


def test_cpp_host_mirror_compiles_against_the_header(tmp_path):
    """The C++ host mirror and its driver build with plain g++ against include/srt_hip.h."""
    import subprocess
    exe = tmp_path / "host_mirror_test"
    subprocess.run(["g++", "-std=c++17", "-O0", "-Wall", "-Werror", "-o", str(exe),
                    os.path.join(ROOT, "tests", "host_mirror_test.cpp"),
                    "-L" + os.path.join(ROOT, "swiftrt_amd", "lib"), "-lSwiftRTHip",
                    "-Wl,-rpath," + os.path.join(ROOT, "swiftrt_amd", "lib")], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode in (0, 2)      # 2: no GPU visible on this host


def test_header_is_plain_c():
    """include/srt_hip.h must be consumable by a C compiler (the Swift importer reads it as C)."""
    import subprocess
    src = '#include "srt_hip.h"\nint main(void){ srtTensorDescriptor d; (void)d; return srtGetVersion() > 0 ? 0 : 1; }\n'
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                    "-x", "c", "-"], input=src, text=True, check=True)
