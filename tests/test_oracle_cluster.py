"""Pins the transformation-compression functions of the CPU oracle (no GPU needed):
  * golden (index, active) recorded from the reference's compiled cluster_forward on
    inputs with exactly representable projections (tests/golden/cluster_golden.npz),
    and the compiled reference itself where oracle/_ref is built;
  * the torch restatement of the reference's own test (tests/test_transformation.py:16-20)
    on such inputs; the known answers count == [0, 513] (bits 0, 8, 24) and the id layout
    idx = [1, 1, 3, 1, 3, 3] with unused clusters;
  * means, mean gradients, reconstruction and its gradient against index_add /
    index_select compositions, torch autograd, and float64 finite differences."""
import os

import numpy as np
import pytest
import torch

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden", "cluster_golden.npz")


def reference_ids(x, w):
    """tests/test_transformation.py:16-20 of the reference, in float64 (exact for the
    integer-valued inputs used here)."""
    h = torch.from_numpy(x).double() @ torch.from_numpy(w).double()
    bits = w.shape[1]
    code = torch.zeros(x.shape[0], dtype=torch.long)
    for i in range(bits):
        code = (code << 1) + (h[:, i] > 0).long()
    unique, inv = torch.unique(code, sorted=True, return_inverse=True)
    idx = inv + 1
    return idx.numpy(), torch.bincount(idx, minlength=unique.numel() + 1).int().numpy(), unique.numel()


def test_lsh_golden_vectors():
    g = np.load(GOLD)
    for i in range(int(g["n_cases"])):
        p = "c%d_" % i
        index, active, _ = oracle.lsh(g[p + "x"], g[p + "w"], int(g[p + "bits"]))
        assert active == int(g[p + "active"])
        assert index.dtype == np.int32 and np.array_equal(index, g[p + "index"])
    index, active, _ = oracle.lsh(g["d_x"], g["d_w"], int(g["d_bits"]))
    assert active == int(g["d_active"]) and np.array_equal(index, g["d_index"])


def test_lsh_matches_compiled_reference_on_exact_inputs():
    ref = pytest.importorskip("compressgnn_runtime_ref")
    rng = np.random.default_rng(8)
    for n, width, bits in [(300, 17, 9), (50, 3, 2), (10, 40, 12)]:
        x = rng.integers(-6, 7, size=(n, width)).astype(np.float32)
        w = rng.integers(-4, 5, size=(width, bits)).astype(np.float32)
        ri, ra = ref.cluster_forward(torch.from_numpy(x), torch.from_numpy(w), bits)
        index, active, _ = oracle.lsh(x, w, bits)
        assert active == ra and np.array_equal(index, ri.numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,width,bits", [(1, 0, 0), (67, 31, 8), (257, 33, 16), (400, 128, 5), (90, 1, 3)])
def test_assign_matches_torch_restatement(dtype, n, width, bits):
    rng = np.random.default_rng(n + bits)
    x = rng.integers(-5, 6, size=(n, width)).astype(dtype)
    w = rng.integers(-3, 4, size=(width, bits)).astype(dtype)
    ids, counts, active = oracle.assign(x, w, bits)
    ri, rc, ra = reference_ids(x, w)
    assert active == ra and np.array_equal(ids, ri) and np.array_equal(counts, rc)
    assert ids.dtype == np.int64 and counts.dtype == np.int32 and counts[0] == 0 and counts.sum() == n


def test_strict_positive_msb_first():
    # h = [0, -0, 3, -2]: only the third plane is strictly positive; column 0 is the MSB
    x = np.array([[1.0]], np.float32)
    w = np.array([[0.0, -0.0, 3.0, -2.0]], np.float32)
    _, _, raw = oracle.lsh(x, w, 4)
    assert raw.tolist() == [0b0010]
    x = np.array([[np.nan]], np.float32)
    _, _, raw = oracle.lsh(x, np.ones((1, 3), np.float32), 3)
    assert raw.tolist() == [0]


@pytest.mark.parametrize("bits", [0, 8, 24])
def test_all_collide_known_answer(bits):
    x = np.ones((513, 33), np.float32)
    w = np.ones((33, bits), np.float32)
    ids, counts, active = oracle.assign(x, w, bits)
    assert active == 1 and counts.tolist() == [0, 513] and set(ids.tolist()) == {1}


def test_empty_input_and_invalid_bits():
    ids, counts, active = oracle.assign(np.zeros((0, 4), np.float32), np.zeros((4, 8), np.float32), 8)
    assert ids.shape == (0,) and counts.tolist() == [0] and active == 0
    with pytest.raises(ValueError):
        oracle.lsh(np.zeros((2, 2), np.float32), np.zeros((2, 31), np.float32), 31)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_mean_and_gradient_closed_forms(dtype):
    rng = np.random.default_rng(2)
    idx = np.array([1, 1, 3, 1, 3, 3], np.int64)
    counts = np.bincount(idx, minlength=5).astype(np.int32)  # clusters 0, 2, 4 unused
    x = rng.standard_normal((6, 5)).astype(dtype)
    reps = oracle.cluster_mean(x, idx, counts)
    xt = torch.from_numpy(x).requires_grad_()
    it = torch.from_numpy(idx)
    ref = torch.zeros(5, 5, dtype=xt.dtype).index_add(0, it, xt) / torch.from_numpy(counts).clamp_min(1).to(xt.dtype)[:, None]
    np.testing.assert_allclose(reps, ref.detach().numpy(), rtol=1e-6, atol=1e-7)
    assert not reps[[0, 2, 4]].any()
    grad = rng.standard_normal((5, 5)).astype(dtype)
    dx = oracle.cluster_mean_backward(grad, idx, counts)
    (want,) = torch.autograd.grad(ref, xt, torch.from_numpy(grad))
    np.testing.assert_allclose(dx, want.numpy(), rtol=1e-6, atol=1e-7)


def test_mean_finite_differences_float64():
    rng = np.random.default_rng(4)
    idx = rng.integers(1, 6, size=30).astype(np.int64)
    counts = np.bincount(idx, minlength=7).astype(np.int32)
    x = rng.standard_normal((30, 3))
    g = rng.standard_normal((7, 3))
    dx = oracle.cluster_mean_backward(g, idx, counts)
    eps = 1e-6
    for (i, k) in [(0, 0), (7, 2), (29, 1)]:
        xp, xm = x.copy(), x.copy()
        xp[i, k] += eps
        xm[i, k] -= eps
        num = ((oracle.cluster_mean(xp, idx, counts) - oracle.cluster_mean(xm, idx, counts)) * g).sum() / (2 * eps)
        assert abs(num - dx[i, k]) < 1e-6


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("width", [1, 31, 128])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("use_bias", [False, True])
def test_reconstruct_and_gradient(dtype, width, relu, use_bias):
    rng = np.random.default_rng(width + relu)
    idx = np.array([1, 1, 3, 1, 3, 3, 0, 4], np.int64)
    reps = rng.standard_normal((5, width)).astype(dtype)
    bias = rng.standard_normal(width).astype(dtype) if use_bias else None
    out = oracle.reconstruct(reps, idx, bias, relu)
    rt_, it = torch.from_numpy(reps).requires_grad_(), torch.from_numpy(idx)
    ref = rt_.index_select(0, it)
    bt = None
    if use_bias:
        bt = torch.from_numpy(bias).requires_grad_()
        ref = ref + bt
    if relu:
        ref = ref.relu()
    assert np.array_equal(out, ref.detach().numpy())
    go = rng.standard_normal(out.shape).astype(dtype)
    rg = oracle.reconstruct_backward(go, idx, out, 5, relu)
    grads = torch.autograd.grad(ref, (rt_, bt) if use_bias else (rt_,), torch.from_numpy(go))
    np.testing.assert_allclose(rg, grads[0].numpy(), rtol=1e-6, atol=1e-6)
    if use_bias:
        np.testing.assert_allclose(rg.sum(0), grads[1].numpy(), rtol=1e-5, atol=1e-5)


def test_relu_mask_uses_saved_output_and_strict_negative_forward():
    # forward: v < 0 -> 0 (so -0.0 stays -0.0); backward: output <= 0 masks the gradient
    reps = np.array([[-1.0, -0.0, 0.0, 2.0]], np.float32)
    idx = np.array([0], np.int64)
    out = oracle.reconstruct(reps, idx, None, True)
    assert out[0, 0] == 0 and np.signbit(out[0, 1]) and out[0, 3] == 2
    rg = oracle.reconstruct_backward(np.ones((1, 4), np.float32), idx, out, 1, True)
    assert rg.tolist() == [[0.0, 0.0, 0.0, 1.0]]
