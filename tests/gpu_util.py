"""Helpers shared by the GPU parity tests (the tests call the C ABI through ratchet_amd's ctypes binding)."""
import numpy as np


def bits(a):
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


def same_bits(a, b):
    """bit equality; any NaN matches any NaN (payloads are not part of the contract)"""
    a, b = np.asarray(a), np.asarray(b)
    if a.dtype.kind == "f":
        return np.all((bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b)))
    return np.array_equal(a, b)


def mismatch_count(a, b):
    a, b = np.asarray(a), np.asarray(b)
    if a.dtype.kind == "f":
        return int(np.count_nonzero(~((bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b)))))
    return int(np.count_nonzero(a != b))


def ulp_diff(a, b):
    """distance in units in the last place between same-typed float arrays; NaN==NaN -> 0, NaN vs number -> huge"""
    a, b = np.asarray(a), np.asarray(b)
    if a.dtype == np.float32:
        it, mask = np.int32, 0x7fffffff
    else:
        it, mask = np.int16, 0x7fff
    def key(x):
        i = x.view(it).astype(np.int64)
        return np.where(i < 0, -(i & mask), i)
    d = np.abs(key(a) - key(b))
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    d = np.where(both_nan, 0, d)
    d = np.where(one_nan, 1 << 40, d)
    return d


def randn(rng, shape, dtype, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float32).astype(dtype)


def describe_mismatch(got, want, x=None, limit=8):
    """human-readable list of the first few differing elements (flat index, input, got, want)"""
    g, w = np.asarray(got).reshape(-1), np.asarray(want).reshape(-1)
    bad = np.flatnonzero(~((bits(g) == bits(w)) | (np.isnan(g) & np.isnan(w))))
    xs = np.asarray(x).reshape(-1) if x is not None and np.asarray(x).size == g.size else None
    rows = []
    for i in bad[:limit]:
        rows.append((int(i), None if xs is None else float(xs[i]), float(g[i]), float(w[i]), hex(int(bits(g)[i])), hex(int(bits(w)[i]))))
    return {"count": int(bad.size), "first": rows}
