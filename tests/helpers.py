"""Shared helpers for the parity tests: seeded inputs, special values, comparisons."""
import numpy as np

SPECIALS = np.array(
    [0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 3.0, -3.0, 6.0, -6.0, 7.5, 88.0, 89.0, -88.0,
     -104.0, -103.5, 100.0, -100.0, 22.0, -22.0, 1e-45, -1e-45, 1.1754942e-38, -1.1754942e-38,
     1.17549435e-38, 3.4028235e38, -3.4028235e38, 1e-30, -1e-30, 1e30, -1e30, np.inf, -np.inf,
     np.nan, 0.70710678, 1.5707964, 3.1415927, -3.1415927, 1e-7, 16777216.0, 0.3, -0.3],
    dtype=np.float32)


def rng(seed):
    return np.random.default_rng(seed)


def normal(seed, shape, sigma=1.0):
    return (rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(sigma)).astype(np.float32)


def uniform(seed, shape, lo, hi):
    u = rng(seed).random(shape, dtype=np.float32)
    return (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float32)


def with_specials(x, seed=0):
    """Scatter the special values over a copy of x (flattened)."""
    x = np.array(x, dtype=np.float32).ravel().copy()
    if x.size >= SPECIALS.size:
        pos = rng(seed + 12345).choice(x.size, SPECIALS.size, replace=False)
        x[pos] = SPECIALS
    return x


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bit_exact(got, want, what=""):
    """Bit-for-bit equality; NaNs are compared by NaN-ness only (sign and payload
    of a NaN are whatever the host's and the device's IEEE propagation give)."""
    got = np.asarray(got, dtype=np.float32).ravel()
    want = np.asarray(want, dtype=np.float32).ravel()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, got.shape, want.shape)
    both_nan = np.isnan(got) & np.isnan(want)
    same = (bits(got) == bits(want)) | both_nan
    if not same.all():
        bad = np.flatnonzero(~same)
        i = bad[0]
        raise AssertionError("%s: %d of %d differ; first at %d: got %r (0x%08x) want %r (0x%08x)" % (
            what, bad.size, got.size, i, got[i], bits(got)[i], want[i], bits(want)[i]))


def assert_rel_close(got, want, rel, what=""):
    """|got - want| <= rel * |want| element-wise (NaN/inf must match exactly)."""
    got = np.asarray(got, dtype=np.float32).ravel()
    want = np.asarray(want, dtype=np.float32).ravel()
    assert got.shape == want.shape
    finite = np.isfinite(want)
    assert (np.isfinite(got) == finite).all(), what + ": finiteness differs"
    g, w = got[finite].astype(np.float64), want[finite].astype(np.float64)
    err = np.abs(g - w)
    ok = err <= rel * np.abs(w)
    if not ok.all():
        i = np.flatnonzero(~ok)[0]
        raise AssertionError("%s: %d of %d outside %g relative; first: got %r want %r" % (
            what, (~ok).sum(), g.size, rel, g[i], w[i]))
    return int((bits(got) != bits(want)).sum())


def ulp_distance(got, want):
    """Distance in units in the last place between two float32 arrays."""
    def key(a):
        u = bits(a).astype(np.int64)
        return np.where(u & 0x80000000, 0x80000000 - u, u)
    return np.abs(key(got) - key(want))
