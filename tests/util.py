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
