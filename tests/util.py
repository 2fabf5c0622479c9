"""Helpers shared by the tests: seeded random CSR blocks and tolerance checks."""
import numpy as np


def random_csr(rng, rows, cols, mean_deg, skew=False, empty_frac=0.2):
    """A random CSR (int64 vlist/elist, float32 values).  skew=True adds a few very
    long rows; a fraction of rows is left empty."""
    deg = rng.poisson(mean_deg, size=rows)
    deg[rng.random(rows) < empty_frac] = 0
    if skew and rows >= 4:
        for r in rng.choice(rows, size=max(1, rows // 50), replace=False):
            deg[r] = int(rng.integers(200, 1500))
    if cols == 0:
        deg[:] = 0
    vlist = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    nnz = int(vlist[-1])
    elist = rng.integers(0, max(cols, 1), size=nnz).astype(np.int64)
    value = rng.standard_normal(nnz).astype(np.float32)
    return vlist, elist, value


def assert_within(a, b, rtol=1e-5, atol=1e-6):
    """|a - b| <= atol + rtol * |b| element-wise (b is the oracle)."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.shape == b.shape, (a.shape, b.shape)
    err = np.abs(a.astype(np.float64) - b.astype(np.float64))
    bound = atol + rtol * np.abs(b.astype(np.float64))
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError("mismatch at %s: got %r want %r (err %.3e, bound %.3e, %d bad of %d)" % (
            i, a[i], b[i], err[i], bound[i], int(bad.sum()), bad.size))
