"""Shared helpers for the parity tests: seeded inputs, storage codecs, error metrics."""
import numpy as np

from oracle import srt_oracle as ora

F32, F16, BF16 = ora.F32, ora.F16, ora.BF16
NP_STORAGE = {F32: np.float32, F16: np.float16, BF16: np.uint16}
# stated tolerances (max-norm relative error against the fp64 GEMM on the same rounded inputs)
TOL = {F32: 1e-5, F16: 2e-2, BF16: 2e-2}
# unit roundoff of the stored result, used for the tighter element-wise bound
ULP = {F32: 2.0 ** -24, F16: 2.0 ** -11, BF16: 2.0 ** -8}


def rng(seed):
    """Counter-based generator (Philox4x32-10) keyed by the config seed."""
    return np.random.Generator(np.random.Philox(seed))


def bf16_encode_fast(x):
    """Vectorised round-to-nearest-even float32 -> bf16 bits (checked against the oracle codec in tests)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = 0x7FFF
    return r


def encode(values, dt):
    """float values -> storage array of element type dt."""
    v = np.asarray(values, dtype=np.float32)
    if dt == F32:
        return v.copy()
    if dt == F16:
        return v.astype(np.float16)
    return bf16_encode_fast(v)


def decode(stored):
    """storage array -> float32 values."""
    if stored.dtype == np.uint16:
        return (stored.astype(np.uint32) << 16).view(np.float32)
    return stored.astype(np.float32)


def to64(stored):
    return decode(stored).astype(np.float64)


def max_norm_rel(c, c64):
    denom = np.max(np.abs(c64))
    return float(np.max(np.abs(c.astype(np.float64) - c64)) / denom) if denom > 0 else 0.0


def elementwise_excess(c, c64, absprod, dt, k):
    """max over elements of |c - c64| / (ulp * |c64| + k * 2^-24 * sum_k |a||b|); <= 1 means every
    element is within one rounding of the stored type plus fp32 accumulation error."""
    bound = ULP[dt] * np.abs(c64) + (k * 2.0 ** -24 + 2.0 ** -20) * absprod + 1e-30
    return float(np.max(np.abs(c.astype(np.float64) - c64) / bound))
