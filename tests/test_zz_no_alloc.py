"""GPU test of srtActivationBackwardBiasNoAlloc: the entry point that takes its workspace from a fixed
device array inside the library instead of the allocator.  Its output must equal
srtActivationBackwardBias's bit for bit (the same kernels run on a different workspace), on two calls
in a row of which the second is smaller, so the array still holds the first call's partial rows when
the second call runs.  Sizes beyond the array's 8 MiB are refused.
"""
import numpy as np
import pytest

import swiftrt_amd as srt
from swiftrt_amd import native
from tests import helpers as H

pytestmark = pytest.mark.gpu


def both_entry_points(y_st, dy_st, act, coef):
    q = srt.current_queue()
    y, dy = srt.Tensor(y_st), srt.Tensor(dy_st)
    outs = []
    for no_alloc in (True, False):
        dx = srt.Tensor(shape=y.shape, dtype=y.dtype)
        db = srt.Tensor(shape=[y.shape[1]], dtype=y.dtype)
        q.activation_backward(y, dy, act, coef, dx, db, no_alloc=no_alloc)
        outs.append((dx.array(), db.array()))
    return outs


@pytest.mark.parametrize("dt", [H.BF16, H.F16, H.F32])
def test_no_alloc_matches_allocating_entry_point_twice_in_a_row(dt):
    g = H.rng(77)
    # a large call first (1024 x 11008: many chunks of partial rows), then a smaller one with a different
    # column count, so that stale rows of the first call lie where the second call's rows go
    for (m, n, act, coef) in [(1024, 11008, srt.ActivationType.relu, 0.0), (300, 520, srt.ActivationType.tanh, 0.0),
                              (70, 123, srt.ActivationType.sigmoid, 0.0)]:
        y_st = H.encode(np.tanh(g.standard_normal((m, n))).astype(np.float32), dt)
        dy_st = H.encode(g.standard_normal((m, n)).astype(np.float32), dt)
        (dx_fixed, db_fixed), (dx_alloc, db_alloc) = both_entry_points(y_st, dy_st, act, coef)
        assert np.array_equal(dx_fixed.view(np.uint8), dx_alloc.view(np.uint8)), (m, n)
        assert np.array_equal(db_fixed.view(np.uint8), db_alloc.view(np.uint8)), (m, n)
        # and the values are the right ones, not merely equal: exact column sums on integer data
    ints = g.integers(-3, 4, (257, 264)).astype(np.float32)
    ones = np.ones_like(ints)
    (dx_fixed, db_fixed), _ = both_entry_points(H.encode(ones, dt), H.encode(ints, dt), srt.ActivationType.identity, 0.0)
    assert np.array_equal(H.decode(dx_fixed), ints)
    assert np.array_equal(H.decode(db_fixed), H.decode(H.encode(ints.sum(axis=0), dt)))


def test_no_alloc_refuses_what_does_not_fit():
    """More than 8 MiB of partial rows: 4 Mi fp32 columns need 16 MiB even as a single chunk."""
    q = srt.current_queue()
    n = 4 << 20
    y = srt.Tensor(np.zeros((1, n), np.float32))
    dx = srt.Tensor(shape=[1, n], dtype=np.float32)
    db = srt.Tensor(shape=[n], dtype=np.float32)
    with pytest.raises(native.SrtError) as e:
        q.activation_backward(y, y, srt.ActivationType.relu, 0.0, dx, db, no_alloc=True)
    assert e.value.status == native.ERROR_INVALID_VALUE
    # without a bias gradient there is no workspace and no limit
    q.activation_backward(y, y, srt.ActivationType.relu, 0.0, dx, None, no_alloc=True)
    # the allocating entry point takes the same problem
    q.activation_backward(y, y, srt.ActivationType.relu, 0.0, dx, db)
    assert np.all(db.array() == 0.0)
