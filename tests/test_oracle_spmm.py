"""Pins the SpMM functions of the CPU oracle (no GPU needed):
  * golden vectors recorded from the reference's own compiled spmm_func
    (tests/golden/spmm_golden.npz) -- bit-exact, incl. accumulate and in-place;
  * the compiled reference itself on fresh random inputs, where oracle/_ref is built;
  * a dense float64 product (catches a transposed operand or a dropped value);
  * the 4-stage compressed chain and its transposed backward against the plain product
    of the uncompressed graph and against the adjoint identity <Ax, g> = <x, A^T g>."""
import os

import numpy as np
import pytest

import oracle
import prep_oracle
from util import random_csr

GOLD = os.path.join(os.path.dirname(__file__), "golden", "spmm_golden.npz")


def test_spmm_golden_vectors():
    g = np.load(GOLD)
    for i in range(int(g["n_cases"])):
        p = "c%d_" % i
        vl, el, va, x = g[p + "vlist"], g[p + "elist"], g[p + "value"], g[p + "x"]
        assert np.array_equal(oracle.spmm(vl, el, va, x), g[p + "fresh"])
        acc = g[p + "base"].copy()
        ret = oracle.spmm(vl, el, va, x, acc)
        assert ret is acc and np.array_equal(acc, g[p + "acc"])
    z = g["ip_z"].copy()
    oracle.spmm(g["ip_vlist"], g["ip_elist"], g["ip_value"], z, z)
    assert np.array_equal(z, g["ip_out"])
    assert np.array_equal(oracle.spmm(g["d_vlist"], g["d_elist"], g["d_value"], g["d_x"]), g["d_fresh"])


def test_spmm_threads_do_not_change_bits():
    rng = np.random.default_rng(3)
    vl, el, va = random_csr(rng, 500, 300, 7.0, skew=True)
    x = rng.standard_normal((300, 19)).astype(np.float32)
    assert np.array_equal(oracle.spmm(vl, el, va, x, None, 1), oracle.spmm(vl, el, va, x, None, 4))


def test_spmm_matches_compiled_reference():
    ref = pytest.importorskip("compressgnn_runtime_ref")
    import torch
    rng = np.random.default_rng(11)
    for rows, cols, F in [(100, 80, 16), (33, 200, 130), (1, 1, 1)]:
        vl, el, va = random_csr(rng, rows, cols, 5.0, skew=rows > 50)
        x = rng.standard_normal((cols, F)).astype(np.float32)
        t = torch.from_numpy
        want = ref.spmm_func(t(vl), t(el), t(va), t(x), "rowbalance", None).numpy()
        assert np.array_equal(oracle.spmm(vl, el, va, x), want)


def test_spmm_dense_float64():
    rng = np.random.default_rng(5)
    rows, cols, F = 60, 45, 11
    vl, el, va = random_csr(rng, rows, cols, 4.0)
    x = rng.standard_normal((cols, F))
    dense = np.zeros((rows, cols))
    for r in range(rows):
        for e in range(vl[r], vl[r + 1]):
            dense[r, el[e]] += va[e]
    got = oracle.spmm(vl, el, va.astype(np.float64), x)
    np.testing.assert_allclose(got, dense @ x, rtol=1e-12, atol=1e-12)


def _compressed_blocks(seed, V=300, freq=3):
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(__file__)), "compressgnn_amd"))
    import compressgnn_offline as off
    v, e = off.gen_copy_model(V, 8.0, 0.7, seed)
    v, e = off.add_self_loop_csr(v, e)
    d = off.get_norm_degree(e, V)
    cv, ce, V, R = off.compress_csr_batch(v, e, 1, 12, freq)
    cv, ce = cv.astype(np.int64), ce.astype(np.int64)
    w = prep_oracle.gcn_norm_csr_compress(cv, ce, d, V, R)
    colptr, row, val = prep_oracle.csc(cv, ce, w, V + R)
    v2v, v2r, r2v, r2r = prep_oracle.hybird_partition(colptr, row, val, V)
    levels, _ = prep_oracle.topo_partition(*r2r)
    fwd = dict(v2v=v2v, v2r=v2r, r2v=r2v, r2r=levels)
    tr = lambda blk, cols: prep_oracle.csc(blk[0], blk[1], blk[2], cols)
    bwd = dict(v2v_t=tr(v2v, V), v2r_t=tr(v2r, R), r2v_t=tr(r2v, V), r2r_t=[tr(lv, R) for lv in levels])
    return (v, e, d), fwd, bwd, V, R


@pytest.mark.parametrize("seed", [0, 1])
def test_compressed_chain_equals_plain_product(seed):
    (v, e, d), fwd, bwd, V, R = _compressed_blocks(seed)
    assert R > 0 and len(fwd["r2r"]) >= 1
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((V, 6))
    to64 = lambda blk: (blk[0], blk[1], blk[2].astype(np.float64))
    fwd64 = dict(v2v=to64(fwd["v2v"]), v2r=to64(fwd["v2r"]), r2v=to64(fwd["r2v"]), r2r=[to64(b) for b in fwd["r2r"]])
    bwd64 = dict(v2v_t=to64(bwd["v2v_t"]), v2r_t=to64(bwd["v2r_t"]), r2v_t=to64(bwd["r2v_t"]),
                 r2r_t=[to64(b) for b in bwd["r2r_t"]])
    out = oracle.compress_spmm_forward(fwd64, x)
    src = np.repeat(np.arange(V), np.diff(v))
    w = d[src].astype(np.float64) * d[e].astype(np.float64)
    plain = np.zeros((V, 6))
    np.add.at(plain, e, w[:, None] * x[src])
    np.testing.assert_allclose(out, plain, rtol=1e-6, atol=1e-7)  # weights are float32 products
    g = rng.standard_normal((V, 6))
    gx = oracle.compress_spmm_backward(bwd64, g)
    plain_t = np.zeros((V, 6))
    np.add.at(plain_t, src, w[:, None] * g[e])
    np.testing.assert_allclose(gx, plain_t, rtol=1e-6, atol=1e-7)
    assert abs((out * g).sum() - (x * gx).sum()) < 1e-9 * max(1.0, abs((out * g).sum()))
