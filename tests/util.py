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


def assert_no_less_accurate(got, sequential, truth, factor=2.0):
    """`got` (the kernel) and `sequential` (the oracle's fp32 sum in the reference's order) are
    two roundings of the same exact result `truth` (float64).  A re-associated sum may differ
    from the sequential one by more than the task's 1e-5/1e-6 on ill-scaled inputs; what must
    hold is that it is no further from the truth: max|got - truth| <= factor * max|sequential -
    truth| (and the same for the mean error, without the factor's slack being needed in
    practice).  Returns (err_got, err_sequential) for the record."""
    got = np.asarray(got, dtype=np.float64)
    seq = np.asarray(sequential, dtype=np.float64)
    truth = np.asarray(truth, dtype=np.float64)
    assert got.shape == seq.shape == truth.shape
    if got.size == 0:
        return 0.0, 0.0
    e_got, e_seq = np.abs(got - truth), np.abs(seq - truth)
    floor = np.finfo(np.float32).eps * max(float(np.abs(truth).max()), 1e-30)  # one ulp of the largest value
    assert e_got.max() <= factor * e_seq.max() + floor, \
        "kernel is %.3e from the float64 result, the sequential fp32 sum %.3e" % (e_got.max(), e_seq.max())
    assert e_got.mean() <= factor * e_seq.mean() + floor, \
        "mean error: kernel %.3e, sequential fp32 sum %.3e" % (e_got.mean(), e_seq.mean())
    # one line for the record (shown with pytest -s)
    print("accuracy vs float64: kernel max %.3e mean %.3e | sequential fp32 max %.3e mean %.3e" % (
        e_got.max(), e_got.mean(), e_seq.max(), e_seq.mean()))
    return float(e_got.max()), float(e_seq.max())
