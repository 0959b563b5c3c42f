"""Helpers shared by the tests."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden(name):
    return dict(np.load(os.path.join(GOLDEN, name + ".npz")))


def rel_err(a, b):
    """max |a-b| over max |b|: the relative error of a tensor against its reference."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    denom = np.max(np.abs(b))
    if denom == 0:
        return float(np.max(np.abs(a)))
    return float(np.max(np.abs(a - b)) / denom)


def assert_close(a, b, tol, what=""):
    e = rel_err(a, b)
    assert e <= tol, "%s: relative error %.3e > %.1e" % (what, e, tol)


def shape_from_geom(oracle, geom):
    n, c, h, w, k, r, s, ph, pw, sh, sw = [int(v) for v in geom]
    return oracle.shape(n, c, h, w, k, r, s, ph, pw, sh, sw)


def to_bf16_bits(a):
    """float32 values that are exactly representable in bfloat16 -> their 16-bit patterns."""
    a = np.ascontiguousarray(a, np.float32)
    bits = a.view(np.uint32)
    assert not np.any(bits & 0xFFFF), "not a bfloat16 value"
    return (bits >> 16).astype(np.uint16)


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def assert_close_bf16(got, want, what="", ulps=1.0):
    """got: bfloat16 results (as float32); want: the unrounded expectation. Each element must lie within
    `ulps` bfloat16 units in the last place of the expectation (half a unit of rounding plus the float
    accumulation error that can push a value across a rounding boundary), relative to its own magnitude,
    with an absolute floor for elements that cancel to nearly zero."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = float(np.max(np.abs(want))) if want.size else 0.0
    with np.errstate(divide="ignore"):
        ulp = np.where(want != 0, 2.0 ** (np.floor(np.log2(np.abs(want) + 1e-300)) - 7), 0.0)  # 8 significant bits
    bound = ulps * ulp + 1e-5 * scale + 1e-30
    bad = np.abs(got - want) > bound
    assert not np.any(bad), "%s: %d of %d elements off by more than %.1f bf16 ulp (worst %.3e vs bound %.3e)" % (
        what, int(bad.sum()), bad.size, ulps, float(np.max(np.abs(got - want) - bound)), float(bound.flat[np.argmax(np.abs(got - want) - bound)]))
