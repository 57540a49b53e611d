"""Comparison helpers shared by the parity tests."""
import numpy as np


def ulp_diff(a, b):
    """Distance in float32 units-in-the-last-place; NaN==NaN, +0 == -0 distance 0."""
    a = np.ascontiguousarray(a, dtype=np.float32).reshape(-1)
    b = np.ascontiguousarray(b, dtype=np.float32).reshape(-1)
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    d = np.where(both_nan, 0, d)
    d = np.where(one_nan, np.iinfo(np.int64).max, d)
    return d


def assert_bits_equal(got, want, what=""):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.shape == want.shape or got.size == want.size, f"{what}: shape {got.shape} vs {want.shape}"
    g = got.reshape(-1).view(np.uint32 if got.dtype == np.float32 else np.uint64)
    w = want.reshape(-1).view(np.uint32 if want.dtype == np.float32 else np.uint64)
    # NaN payloads may differ between libm and the GPU; compare NaN-ness there
    nan = np.isnan(got.reshape(-1)) & np.isnan(want.reshape(-1))
    bad = (g != w) & ~nan
    if bad.any():
        i = int(np.flatnonzero(bad)[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {g.size} elements differ; first at {i}: "
                             f"got {got.reshape(-1)[i]!r} want {want.reshape(-1)[i]!r}")


def rel_frobenius(got, ref64):
    got = np.asarray(got, dtype=np.float64)
    ref64 = np.asarray(ref64, dtype=np.float64)
    den = np.linalg.norm(ref64.reshape(-1))
    return np.linalg.norm((got - ref64).reshape(-1)) / (den if den > 0 else 1.0)
