"""Parity of the transformation-compression kernels (through the C ABI) against the
CPU oracle, on the grid of the reference's own test (tests/test_transformation.py:21-39):
dtype x width x (n, bits).  Ids, counts, the active-bucket count, mean gradients and
reconstructions are bit-exact.  Cluster sums (means, reconstruct gradients) are
bit-exact for clusters of at most 64 members (one run of the segmented reduction) and
within the reference test's own tolerance (atol 1e-5, rtol 1e-4 for float32,
tests/test_transformation.py:14) for larger ones, whose sums are re-associated."""
import numpy as np
import pytest
import torch

import oracle
from compressgnn_amd import abi
from util import assert_no_less_accurate, assert_within

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {np.float32: dict(rtol=1e-4, atol=1e-5), np.float64: dict(rtol=1e-12, atol=1e-13)}


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def pack_signs(out):
    """The sign words of cgnn_reconstruct_signs from the rows: bit f % 32 of word f // 32 is set
    unless out[i, f] <= 0 (so a NaN keeps its bit, as it keeps its gradient in the reference's mask,
    cluster_kernel.cu:98-108); bits past the width are clear."""
    n, width = out.shape
    words = (width + 31) // 32
    bits = np.zeros((n, words * 32), dtype=np.uint64)
    bits[:, :width] = ~(out <= 0)
    packed = (bits.reshape(n, words, 32) << np.arange(32, dtype=np.uint64)).sum(axis=2)
    return packed.astype(np.uint32).view(np.int32)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("width", [0, 1, 31, 33, 100, 128, 602])
@pytest.mark.parametrize("n,bits", [(1, 0), (67, 8), (257, 16), (1000, 5), (5000, 12), (300, 20)])
def test_assign_mean_reconstruct(dtype, width, n, bits):
    rng = np.random.default_rng(1000 * bits + width + n)
    x = rng.standard_normal((n, width)).astype(dtype)
    w = rng.standard_normal((width, bits)).astype(dtype)
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    ids, counts, active = abi.lsh_assign(_t(x), _t(w), bits)
    torch.cuda.synchronize()
    assert active == want_active
    assert ids.dtype == torch.int64 and counts.dtype == torch.int32
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.array_equal(counts.cpu().numpy(), want_counts)
    if width == 0:
        return
    groups = active + 1
    members = abi.cluster_members(ids, groups)
    offsets, perm, sorted_id = (m.cpu().numpy() for m in members)
    order = np.argsort(want_ids, kind="stable")
    assert np.array_equal(perm, order.astype(np.int32))
    assert np.array_equal(sorted_id, want_ids[order].astype(np.int32))
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(want_counts)]).astype(np.int32))
    tol = TOL[dtype]
    small = want_counts <= 64
    reps = abi.cluster_mean(_t(x), members, counts).cpu().numpy()
    want_reps = oracle.cluster_mean(x, want_ids, want_counts)
    assert_within(reps, want_reps, **tol)
    assert np.array_equal(reps[small], want_reps[small])
    grad = rng.standard_normal((groups, width)).astype(dtype)
    want_dx = oracle.cluster_mean_backward(grad, want_ids, want_counts)
    assert np.array_equal(abi.cluster_mean_backward(_t(grad), ids, counts).cpu().numpy(), want_dx)
    assert np.array_equal(abi.cluster_mean_backward(_t(grad), ids, counts, members).cpu().numpy(), want_dx)
    bias = rng.standard_normal(width).astype(dtype)
    for relu in (False, True):
        for b in (None, bias):
            out = abi.reconstruct(_t(grad), ids, None if b is None else _t(b), relu)
            want = oracle.reconstruct(grad, want_ids, b, relu)
            assert np.array_equal(out.cpu().numpy(), want)
            grouped = abi.reconstruct(_t(grad), ids, None if b is None else _t(b), relu, members)
            assert np.array_equal(grouped.cpu().numpy(), want)  # row order does not change the result
            go = rng.standard_normal((n, width)).astype(dtype)
            rg = abi.reconstruct_backward(_t(go), out, members, groups, relu).cpu().numpy()
            want_rg = oracle.reconstruct_backward(go, want_ids, want, groups, relu)
            assert_within(rg, want_rg, **tol)
            assert np.array_equal(rg[small], want_rg[small])
            if relu:
                # the same pair with the mask as one bit per element: same rows, the bits of the rows,
                # and the very sums of the form that reads the rows back
                for m in (None, members):
                    rows, signs = abi.reconstruct_signs(_t(grad), ids, None if b is None else _t(b), m)
                    assert np.array_equal(rows.cpu().numpy(), want)
                    assert signs.shape == (n, (width + 31) // 32) and signs.dtype == torch.int32
                    assert np.array_equal(signs.cpu().numpy(), pack_signs(want))
                rg_bits = abi.reconstruct_backward_signs(_t(go), signs, members, groups).cpu().numpy()
                assert np.array_equal(rg_bits, rg)


@pytest.mark.parametrize("width,bits", [
    (4, 3), (16, 16), (20, 9), (48, 17), (64, 30), (84, 12), (100, 16), (100, 24), (104, 16), (112, 7),
    (124, 16), (128, 16), (128, 30), (132, 16), (256, 16), (300, 21), (512, 8), (37, 16), (130, 19)])
def test_assign_shapes(width, bits):
    """Ids and counts over the widths that select the different projection kernels
    (whole-row tiles with 1..32 packs per row, padded and unpadded LDS strides, several
    passes per tile, unaligned widths) and both plane-group counts, on enough rows
    (100k + a partial tile) that every persistent wave walks several tiles."""
    n = 100_003
    rng = np.random.default_rng(width * 100 + bits)
    x = rng.standard_normal((n, width)).astype(np.float32)
    w = rng.standard_normal((width, bits)).astype(np.float32)
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    ids, counts, active = abi.lsh_assign(_t(x), _t(w), bits)
    torch.cuda.synchronize()
    assert active == want_active
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.array_equal(counts.cpu().numpy(), want_counts)


@pytest.mark.parametrize("width,bits", [(100, 16), (64, 16), (128, 20)])
def test_assign_many_tiles_a_wave(width, bits):
    """A million rows: every wave of the projection kernel takes some six to ten tiles from
    its workgroup's queue (six, eight and four waves a workgroup at these widths); ids and
    counts against the oracle, bit for bit."""
    n = 1_000_003
    rng = np.random.default_rng(width + bits)
    x = rng.standard_normal((n, width)).astype(np.float32)
    w = rng.standard_normal((width, bits)).astype(np.float32)
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    ids, counts, active = abi.lsh_assign(_t(x), _t(w), bits)
    torch.cuda.synchronize()
    assert active == want_active
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.array_equal(counts.cpu().numpy(), want_counts)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("width", [8, 12, 16, 20, 36, 100, 132])
@pytest.mark.parametrize("n", [63, 64, 65, 1025, 20011])
def test_gathers_over_rows_that_are_not_whole_lines(dtype, width, n):
    """Mean gradient and reconstruct in natural row order at widths whose rows are 16-byte
    packs but not whole 128-byte lines: the output is then produced pack by pack, 64 rows or
    a multiple of 64 a workgroup; row counts on both sides of those bounds, bit for bit
    against the oracle."""
    rng = np.random.default_rng(width * 100003 + n)
    groups = 1 + min(n, 97)
    ids_np = rng.integers(1, groups, size=n).astype(np.int64) if groups > 1 else np.zeros(n, np.int64)
    counts_np = np.bincount(ids_np, minlength=groups).astype(np.int32)
    ids, counts = torch.from_numpy(ids_np).to(DEV), torch.from_numpy(counts_np).to(DEV)
    grad = rng.standard_normal((groups, width)).astype(dtype)
    want_dx = oracle.cluster_mean_backward(grad, ids_np, counts_np)
    assert np.array_equal(abi.cluster_mean_backward(_t(grad), ids, counts).cpu().numpy(), want_dx)
    bias = rng.standard_normal(width).astype(dtype)
    for relu in (False, True):
        for b in (None, bias):
            out = abi.reconstruct(_t(grad), ids, None if b is None else _t(b), relu)
            assert np.array_equal(out.cpu().numpy(), oracle.reconstruct(grad, ids_np, b, relu))


@pytest.mark.parametrize("shape", ["uniform", "one_code", "few_codes", "relu"])
@pytest.mark.parametrize("bits", [1, 8, 16, 23])
def test_grouped_assign_matches_counter_path(shape, bits):
    """cgnn_lsh_group (sort of the codes) against cgnn_lsh_hash/scan/finish (bucket
    counters) + cgnn_cluster_members and against the oracle, on code distributions from
    uniform to everything in one code: ids, counts, active and member lists are identical."""
    rng = np.random.default_rng(bits * 7 + len(shape))
    n, width = 70_001, 24
    x = rng.standard_normal((n, width)).astype(np.float32)
    if shape == "one_code":
        x[:] = x[0]
    elif shape == "few_codes":
        x = x[rng.integers(0, 5, size=n) ** 2 % 7]
    elif shape == "relu":
        x = np.maximum(x - 1.0, 0).astype(np.float32)
    w = rng.standard_normal((width, bits)).astype(np.float32)
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    ids0, counts0, active0 = abi.lsh_assign(_t(x), _t(w), bits)
    members0 = abi.cluster_members(ids0, active0 + 1)
    ids, counts, active, members = abi.lsh_assign_grouped(_t(x), _t(w), bits)
    torch.cuda.synchronize()
    assert active == active0 == want_active
    assert np.array_equal(ids.cpu().numpy(), want_ids) and torch.equal(ids, ids0)
    assert np.array_equal(counts.cpu().numpy(), want_counts) and torch.equal(counts, counts0)
    for got, ref in zip(members[:3], members0):
        assert got.dtype == ref.dtype and torch.equal(got, ref)
    assert members[3] == int(want_counts.max())


def test_grouped_assign_empty():
    ids, counts, active, members = abi.lsh_assign_grouped(torch.zeros(0, 8, device=DEV), torch.randn(8, 8, device=DEV), 8)
    assert ids.numel() == 0 and active == 0 and counts.tolist() == [0] and members[0].tolist() == [0, 0]
    assert members[3] == 0


def test_assign_denormal_and_cancelling_projections():
    """Projections that end exactly at zero, in the denormal range or one ulp from zero
    decide bits by the last rounding: the chains must be fused multiply-adds."""
    rng = np.random.default_rng(11)
    n, width, bits = 4096, 8, 16
    x = rng.standard_normal((n, width)).astype(np.float32)
    w = rng.standard_normal((width, bits)).astype(np.float32)
    x[:, 4:] = -x[:, :4]          # second half cancels the first when the planes repeat
    w[4:, :8] = w[:4, :8]         # planes 0..7: exact cancellation -> h == 0 -> bit 0
    w[4:, 8:] = np.nextafter(w[:4, 8:], np.float32(np.inf))  # planes 8..15: residue of one ulp
    x[::3] *= np.float32(1e-22)   # products deep in the denormal range
    want_ids, want_counts, want_active = oracle.assign(x, w, bits)
    ids, counts, active = abi.lsh_assign(_t(x), _t(w), bits)
    assert active == want_active
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.array_equal(counts.cpu().numpy(), want_counts)


@pytest.mark.parametrize("bits", [0, 8, 24])
def test_all_collide(bits):
    """Known answer of the reference's test: every row in one bucket -> count == [0, 513]."""
    x = torch.ones(513, 33, device=DEV)
    w = torch.ones(33, bits, device=DEV)
    ids, counts, active = abi.lsh_assign(x, w, bits)
    assert active == 1 and counts.tolist() == [0, 513]
    assert ids.unique().tolist() == [1]


def test_empty_input():
    x = torch.zeros(0, 8, device=DEV)
    w = torch.randn(8, 8, device=DEV)
    ids, counts, active = abi.lsh_assign(x, w, 8)
    assert ids.numel() == 0 and active == 0 and counts.tolist() == [0]


def test_ids_match_exact_integer_projection():
    """Independent of any summation order: integer-valued data make every projection
    exact, so the ids must equal those of a float64 matmul (the torch restatement in
    the reference's test, tests/test_transformation.py:16-20)."""
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, size=(4000, 37)).astype(np.float32)
    w = rng.integers(-3, 4, size=(37, 11)).astype(np.float32)
    h = x.astype(np.float64) @ w.astype(np.float64)
    code = np.zeros(len(x), np.int64)
    for j in range(11):
        code = (code << 1) + (h[:, j] > 0)
    uniq, inv = np.unique(code, return_inverse=True)
    ids, counts, active = abi.lsh_assign(_t(x), _t(w), 11)
    assert active == len(uniq)
    assert np.array_equal(ids.cpu().numpy(), inv + 1)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(inv + 1, minlength=len(uniq) + 1))


def test_large_cluster_sums():
    """A few hot clusters (tens of thousands of members): rows of the member CSR span
    hundreds of runs."""
    rng = np.random.default_rng(9)
    n, F = 60000, 100
    ids_np = rng.choice([1, 2, 3, 7], size=n, p=[0.6, 0.3, 0.09, 0.01]).astype(np.int64)
    counts_np = np.bincount(ids_np, minlength=9).astype(np.int32)
    x = rng.standard_normal((n, F)).astype(np.float32)
    ids, counts = _t(ids_np), _t(counts_np)
    members = abi.cluster_members(ids, 9)
    reps = abi.cluster_mean(_t(x), members, counts).cpu().numpy()
    want64 = oracle.cluster_mean(x.astype(np.float64), ids_np, counts_np)
    np.testing.assert_allclose(reps, want64, rtol=1e-5, atol=1e-6)
    again = abi.cluster_mean(_t(x), members, counts).cpu().numpy()
    assert np.array_equal(reps, again)
    # with the size of the largest group given, the chains of carries are known to be
    # short enough for the serial fix-up alone; a wrong (too small) hint only costs time
    largest = int(counts_np.max())
    hinted = abi.cluster_mean(_t(x), members, counts, max_members=largest).cpu().numpy()
    np.testing.assert_allclose(hinted, want64, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(abi.cluster_mean(_t(x), members, counts, max_members=1).cpu().numpy(), want64,
                               rtol=1e-5, atol=1e-6)
    out = rng.standard_normal((n, F)).astype(np.float32)
    go = rng.standard_normal((n, F)).astype(np.float32)
    rg = abi.reconstruct_backward(_t(go), _t(out), members, 9, True).cpu().numpy()
    want = oracle.reconstruct_backward(go.astype(np.float64), ids_np, out.astype(np.float64), 9, True)
    # Sums of up to 18,000 N(0,1) terms (magnitude ~130): two fp32 summation orders differ by
    # ~1e-4 absolute, beyond the reference test's atol of 1e-5.  The bar that can fail: the
    # kernel is no further from the float64 sums than the oracle's sequential fp32 scatter-add.
    sequential = oracle.reconstruct_backward(go, ids_np, out, 9, True)
    assert_no_less_accurate(rg, sequential, want, factor=1.5)
    np.testing.assert_allclose(rg, want, rtol=1e-4, atol=1e-3)
    # the means of the same clusters: unnormalised sums are as large, the quotient is small
    assert_no_less_accurate(reps, oracle.cluster_mean(x, ids_np, counts_np), want64, factor=1.5)


def test_sign_bits_of_special_values():
    """Zero of either sign drops the gradient, NaN and the smallest denormal keep it: the mask
    `output <= 0` of the reference (cluster_kernel.cu:98-108), bit by bit."""
    specials = np.array([0.0, -0.0, np.nan, 1e-45, -1e-45, np.inf, -np.inf, 1.0], dtype=np.float32)
    width = 70
    reps = np.resize(specials, (3, width)).astype(np.float32)
    reps[1] = np.roll(reps[0], 3)
    reps[2] = -reps[0]
    ids = np.array([2, 0, 1, 1, 0, 2, 2], dtype=np.int64)
    want = oracle.reconstruct(reps, ids, None, True)
    rows, signs = abi.reconstruct_signs(_t(reps), _t(ids), None, None)
    assert np.array_equal(rows.cpu().numpy(), want, equal_nan=True)
    assert np.array_equal(signs.cpu().numpy(), pack_signs(want))
    members = abi.cluster_members(_t(ids), 3)
    go = np.random.default_rng(3).standard_normal((7, width)).astype(np.float32)
    got = abi.reconstruct_backward_signs(_t(go), signs, members, 3).cpu().numpy()
    assert np.array_equal(got, oracle.reconstruct_backward(go, ids, want, 3, True))


def test_memory_probes_move_what_they_say():
    """The calibration kernels: the copy reproduces its source, the fill writes zeros over exactly n bytes."""
    import ctypes
    L = abi.lib()
    n = 16 * 100003
    src = torch.randint(1, 255, (n + 16,), dtype=torch.uint8, device=DEV)
    dst = torch.full((n + 16,), 7, dtype=torch.uint8, device=DEV)
    abi.check(L.cgnn_copy_bytes(abi.ptr(src), abi.ptr(dst), ctypes.c_size_t(n), abi.stream_of(src)))
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src[:n]) and bool((dst[n:] == 7).all())
    abi.check(L.cgnn_fill_bytes(abi.ptr(dst), ctypes.c_size_t(n), abi.stream_of(dst)))
    torch.cuda.synchronize()
    assert int(dst[:n].count_nonzero()) == 0 and bool((dst[n:] == 7).all())
    sink = torch.zeros(1, dtype=torch.int32, device=DEV)
    abi.check(L.cgnn_read_bytes(abi.ptr(src), ctypes.c_size_t(n), abi.ptr(sink), abi.stream_of(src)))
    torch.cuda.synchronize()
    assert L.cgnn_fill_bytes(abi.ptr(dst), ctypes.c_size_t(7), abi.stream_of(dst)) != 0


def test_reference_signature_operators_read_the_host_once_per_index():
    """The operators called with the reference's own argument lists (index and nothing else,
    src/runtime/csrc/cluster/cluster_ops.h:5-13): the reference reads the host once per assignment
    (cluster_kernel.cu:147) and never in mean / reconstruct.  Here the ids that cluster_assign
    returned are known to the operators (no read at all), an index from elsewhere is checked on
    its first use only, and an index that was written to since is checked again.  Host reads are
    caught by torch's synchronisation check (any .item() / .cpu() of a device tensor raises)."""
    import compressgnn_runtime as rt
    rng = np.random.default_rng(4)
    n, F, Fo, bits = 30000, 40, 24, 9
    xn = rng.standard_normal((n, F)).astype(np.float32)
    pl = rng.standard_normal((F, bits)).astype(np.float32)
    x, planes = torch.from_numpy(xn).to(DEV), torch.from_numpy(pl).to(DEV)
    ids, counts, active = rt.cluster_assign(x, planes, bits, rt.cluster_workspace(x, bits))
    groups = active + 1
    hidden = torch.from_numpy(rng.standard_normal((groups, Fo)).astype(np.float32)).to(DEV)
    bias = torch.from_numpy(rng.standard_normal(Fo).astype(np.float32)).to(DEV)
    go = torch.from_numpy(rng.standard_normal((n, Fo)).astype(np.float32)).to(DEV)
    gr = torch.from_numpy(rng.standard_normal((groups, F)).astype(np.float32)).to(DEV)

    def chain(index):
        reps = rt.cluster_mean(x, index, counts)
        out = rt.cluster_reconstruct(hidden, index, bias, True)
        rg = rt.cluster_reconstruct_backward(go, index, out, groups, True)
        dx = rt.cluster_mean_backward(gr, index, counts)
        return reps, out, rg, dx

    def without_host_reads(fn):
        torch.cuda.synchronize()
        torch.cuda.set_sync_debug_mode("error")
        try:
            return fn()
        finally:
            torch.cuda.set_sync_debug_mode("default")

    # the check does catch a host read
    with pytest.raises(RuntimeError):
        without_host_reads(lambda: counts.sum().item())
    got = without_host_reads(lambda: chain(ids))
    ids_np, counts_np = ids.cpu().numpy(), counts.cpu().numpy()
    want_reps = oracle.cluster_mean(xn, ids_np, counts_np)
    want_out = oracle.reconstruct(hidden.cpu().numpy(), ids_np, bias.cpu().numpy(), True)
    assert_within(got[0].cpu().numpy(), want_reps, rtol=1e-4, atol=1e-5)
    assert np.array_equal(got[1].cpu().numpy(), want_out)
    assert_within(got[2].cpu().numpy(), oracle.reconstruct_backward(go.cpu().numpy(), ids_np, want_out, groups, True), rtol=1e-4, atol=1e-5)
    assert np.array_equal(got[3].cpu().numpy(), oracle.cluster_mean_backward(gr.cpu().numpy(), ids_np, counts_np))
    # an index from elsewhere: checked on first use (gather first, then a reduction), silent afterwards
    for first in (lambda i: rt.cluster_reconstruct(hidden, i, bias, True), lambda i: rt.cluster_mean(x, i, counts)):
        foreign = ids.clone()
        first(foreign)
        again = without_host_reads(lambda: chain(foreign))
        for a, b in zip(again, got):
            assert torch.equal(a, b)
        # written to since: no longer trusted, and the bad id is reported
        foreign[17] = groups + 5
        with pytest.raises(RuntimeError, match="outside"):
            rt.cluster_reconstruct(hidden, foreign, bias, True)
        with pytest.raises(RuntimeError, match="outside"):
            rt.cluster_mean(x, foreign, counts)
