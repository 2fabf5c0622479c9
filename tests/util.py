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


def closed_form_transpose(vlist, elist, value, cols):
    """CSR -> CSC as mathematics fixes it: a stable sort of the entries by column (ties keep
    storage order, which is what SparseTensor.csc() gives).  No product code involved."""
    vlist, elist = np.asarray(vlist, np.int64), np.asarray(elist, np.int64)
    order = np.argsort(elist, kind="stable")
    rowidx = np.repeat(np.arange(len(vlist) - 1, dtype=np.int64), np.diff(vlist))
    colptr = np.concatenate([[0], np.cumsum(np.bincount(elist, minlength=cols))]).astype(np.int64)
    return colptr, rowidx[order], (None if value is None else np.asarray(value)[order])


def expand_compressed_rows(out_ptr, out_col, V):
    """The vertex rows of a compressed CSR (rows V.. are rules) with every rule replaced by its
    children, recursively, in place and in order.  Returns (rowptr, columns) of the expansion."""
    out_ptr, out_col = np.asarray(out_ptr, np.int64), np.asarray(out_col, np.int64)
    rule_ptr = out_ptr[V:] - out_ptr[V]
    rule_col = out_col[out_ptr[V]:]
    rule_len = np.diff(rule_ptr)
    col = out_col[:out_ptr[V]].copy()
    row = np.repeat(np.arange(V, dtype=np.int64), np.diff(out_ptr[:V + 1]))
    for _ in range(64):
        is_rule = col >= V
        if not is_rule.any():
            break
        lens = np.where(is_rule, rule_len[np.where(is_rule, col - V, 0)], 1)
        start = np.concatenate([[0], np.cumsum(lens)])
        new_row = np.repeat(row, lens)
        within = np.arange(start[-1]) - np.repeat(start[:-1], lens)
        src_rule = np.repeat(np.where(is_rule, col - V, 0), lens)
        from_rule = np.repeat(is_rule, lens)
        new_col = np.where(from_rule, rule_col[np.minimum(rule_ptr[src_rule] + within, max(len(rule_col) - 1, 0))]
                           if len(rule_col) else 0, np.repeat(col, lens))
        col, row = new_col, new_row
    else:
        raise AssertionError("rules nest deeper than 64 levels (a cycle?)")
    rowptr = np.concatenate([[0], np.cumsum(np.bincount(row, minlength=V))]).astype(np.int64)
    return rowptr, col


def assert_compression_contract(vlist, elist, got):
    """What the reference's tests pin at the compressor boundary
    (tests/test_batch_compression.py:15-36,52-55, tests/test_offline_compression.py:7-25): int32
    arrays, a well-formed CSR over V + R rows, every child of a rule has a smaller id than the
    rule, and every vertex row expands to exactly the input row, in order."""
    out_ptr, out_col, V, R = got
    vlist, elist = np.asarray(vlist, np.int64), np.asarray(elist, np.int64)
    assert out_ptr.dtype == np.int32 and out_col.dtype == np.int32
    assert V == len(vlist) - 1 and len(out_ptr) == V + R + 1
    assert out_ptr[0] == 0 and out_ptr[-1] == len(out_col) and (np.diff(out_ptr) >= 0).all()
    if len(out_col):
        assert out_col.min() >= 0 and out_col.max() < V + R
    if R:
        rule_rows = np.repeat(np.arange(V, V + R), np.diff(out_ptr[V:]))
        assert (out_col[out_ptr[V]:] < rule_rows).all(), "a rule refers to itself or to a later rule"
        assert (np.diff(out_ptr[V:]) >= 2).all(), "a rule with fewer than two children"
    rowptr, col = expand_compressed_rows(out_ptr, out_col, V)
    assert np.array_equal(rowptr, vlist - vlist[0]) and np.array_equal(col, elist)
