"""Host logic of Compressgnn_Cluster / Compressgnn_Reconstruct (refresh schedule, cache
namespaces and invalidation, loss-driven interval, argument errors) -- the behavioural
checks of the reference's tests/test_transformation.py:58-107, run on CPU tensors with
the native operators replaced by the CPU oracle (the product has no CPU operators; this
stand-in exists only in this test)."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [os.path.join(ROOT, "compressgnn_amd"), os.path.join(ROOT, "compressgnn_amd", "layer"),
                os.path.join(ROOT, "compressgnn_amd", "loader")]

import oracle  # noqa: E402
import CompressgnnCluster as cc  # noqa: E402
from CompressgnnCluster import Compressgnn_Cluster, Compressgnn_Cluster_Function  # noqa: E402
from CompressgnnReconstruct import Compressgnn_Reconstruct  # noqa: E402


class OracleNative:
    """compressgnn_runtime's cluster operators on CPU tensors, computed by the oracle."""
    calls = 0

    @staticmethod
    def cluster_workspace(x, bits):
        return []

    @classmethod
    def cluster_assign(cls, x, planes, bits, workspace):
        if planes.shape != (x.shape[1], bits):
            raise RuntimeError("Hash plane shape/device/dtype mismatch")
        cls.calls += 1
        ids, counts, active = oracle.assign(x.detach().numpy(), planes.detach().numpy(), bits)
        return torch.from_numpy(ids), torch.from_numpy(counts), active

    @classmethod
    def cluster_assign_members(cls, x, planes, bits):
        index, counts, active = cls.cluster_assign(x, planes, bits, None)
        return index, counts, active, cls.cluster_members(index, active + 1)

    @staticmethod
    def cluster_members(index, groups):
        order = np.argsort(index.numpy(), kind="stable")
        return [torch.zeros(groups + 1, dtype=torch.int32), torch.from_numpy(order.astype(np.int32)),
                torch.from_numpy(index.numpy()[order].astype(np.int32))]

    @staticmethod
    def cluster_mean(x, index, counts, members=None):
        return torch.from_numpy(oracle.cluster_mean(x.detach().numpy(), index.numpy(), counts.numpy()))

    @staticmethod
    def cluster_mean_backward(grad, index, counts, members=None):
        return torch.from_numpy(oracle.cluster_mean_backward(grad.numpy(), index.numpy(), counts.numpy()))


@pytest.fixture(autouse=True)
def oracle_native(monkeypatch):
    monkeypatch.setattr(cc, "_native", OracleNative)
    yield


def scatter_mean(x, index, groups):
    s = torch.zeros(groups, x.size(1), dtype=x.dtype).index_add_(0, index, x)
    return s / torch.bincount(index, minlength=groups).clamp_min(1).to(x.dtype)[:, None]


def close(a, b):
    torch.testing.assert_close(a, b, atol=1e-5, rtol=1e-4)


def test_refresh_schedule_and_current_gradients():
    torch.manual_seed(26)
    c = Compressgnn_Cluster(7, 4, refresh_interval=5)
    ptr = None
    for epoch in range(12):
        x = torch.randn(19, 7, requires_grad=True)
        out, index = c(x, epoch=epoch, cache_key='graph-A')
        assert c.last_refreshed == (epoch % 5 == 0)
        if epoch % 5:
            assert index.data_ptr() == ptr
        ptr = index.data_ptr()
        ref = scatter_mean(x, index, out.size(0))
        close(out, ref)
        close(torch.autograd.grad(out.square().sum(), x)[0], torch.autograd.grad(ref.square().sum(), x)[0])
    assert c.refresh_count == 3


def test_cache_namespaces_and_invalidation():
    torch.manual_seed(1)
    c = Compressgnn_Cluster(7, 4, refresh_interval=5)
    c.set_epoch(0)
    x = torch.randn(19, 7)
    _, train_index = c(x)
    train_ptr = train_index.data_ptr()
    c.eval()
    _, eval_index = c(-x)
    assert eval_index.data_ptr() != train_ptr
    c.train()
    _, index = c(x, epoch=1)
    assert not c.last_refreshed and index.data_ptr() == train_ptr
    c(x, epoch=1, cache_key='different-order')
    assert c.last_refreshed
    c(torch.randn(20, 7), epoch=1)
    assert c.last_refreshed
    c(x, epoch=1)
    c.random_vectors.add_(.01)
    c(x, epoch=1)
    assert c.last_refreshed
    c.load_state_dict(c.state_dict())
    c(x, epoch=1)
    assert c.last_refreshed
    c.double()
    c(x.double(), epoch=1)
    assert c.last_refreshed
    c(x.double(), epoch=1, force_refresh=True)
    assert c.last_refreshed
    # going back in time resets the cache
    c.set_epoch(0)
    c(x.double())
    assert c.last_refreshed
    # cache disabled: every call refreshes
    n = Compressgnn_Cluster(7, 4, cache=False)
    n(x, epoch=0)
    n(x, epoch=0)
    assert n.refresh_count == 2


def test_saved_assignment_survives_later_refresh():
    torch.manual_seed(2)
    c = Compressgnn_Cluster(7, 4, refresh_interval=5)
    a = torch.randn(19, 7, requires_grad=True)
    b = torch.randn(19, 7, requires_grad=True)
    ya, ia = c(a, epoch=5)
    yb, ib = c(b, epoch=10)
    ra, rb = scatter_mean(a, ia, ya.size(0)), scatter_mean(b, ib, yb.size(0))
    ga = torch.autograd.grad(ya.square().sum() + yb.square().sum(), (a, b))
    gb = torch.autograd.grad(ra.square().sum() + rb.square().sum(), (a, b))
    close(ga[0], gb[0])
    close(ga[1], gb[1])


def test_shared_transforms_then_reconstruct():
    torch.manual_seed(3)
    c = Compressgnn_Cluster(7, 4, refresh_interval=5)
    reconstruct = Compressgnn_Reconstruct()
    layers = torch.nn.Sequential(torch.nn.Linear(7, 9), torch.nn.ReLU(), torch.nn.Linear(9, 3))
    x = torch.randn(19, 7, requires_grad=True)
    rep, ii = c(x, epoch=15)
    out = reconstruct(layers(rep), ii)  # CPU tensors take the index_select composition
    ref = layers(scatter_mean(x, ii, rep.size(0))).index_select(0, ii)
    close(out, ref)
    params = [x] + list(layers.parameters())
    for g1, g2 in zip(torch.autograd.grad(out.square().sum(), params), torch.autograd.grad(ref.square().sum(), params)):
        close(g1, g2)
    out = reconstruct(rep, ii, bias=torch.ones(7), activation='relu')
    close(out, (rep.index_select(0, ii) + 1).relu())
    with pytest.raises(ValueError):
        reconstruct(rep, ii, activation='tanh')


def test_epoch_required_and_loss_policy():
    c = Compressgnn_Cluster(7, 4, refresh_interval=5)
    with pytest.raises(ValueError):
        c(torch.zeros(10, 7))
    a = Compressgnn_Cluster(7, 4, refresh_policy='loss', q_min=1, q_max=10, tau_loss=.1)
    a.set_epoch(0, loss=1.)
    a.set_epoch(1, loss=1.)
    assert a.current_interval == 10
    a.set_epoch(2, loss=2.)
    assert a.current_interval == 1
    with pytest.raises(TypeError):
        a.set_epoch(3, loss=torch.tensor(1.))
    with pytest.raises(ValueError):
        a.set_epoch(3, loss=float('nan'))
    with pytest.raises(ValueError):
        a.set_epoch(-1)


def test_constructor_and_input_errors():
    for invalid in [-1, 31]:
        with pytest.raises(ValueError):
            Compressgnn_Cluster(7, invalid)
    with pytest.raises(ValueError):
        Compressgnn_Cluster(7, 4, refresh_interval=0)
    with pytest.raises(ValueError):
        Compressgnn_Cluster(7, 4, refresh_policy='sometimes')
    with pytest.raises(ValueError):
        Compressgnn_Cluster(7, 4, refresh_policy='loss')
    c = Compressgnn_Cluster(7, 4)
    with pytest.raises(ValueError):
        c(torch.zeros(3, 8))
    with pytest.raises(ValueError):
        c(torch.zeros(3, 7, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        cc._assign(torch.zeros(3, 7), torch.zeros(7, 3), 4)


def test_legacy_entry_and_return_contracts():
    torch.manual_seed(4)
    a = Compressgnn_Cluster(7, 4)
    x = torch.randn(10, 7, requires_grad=True)
    y, ii, active = Compressgnn_Cluster_Function.apply(x, a.random_vectors, 4, True)
    ref = scatter_mean(x, ii, active + 1)
    close(y, ref)
    close(torch.autograd.grad(y.sum(), x)[0], torch.autograd.grad(ref.sum(), x)[0])
    only = Compressgnn_Cluster(7, 4, training=False)
    out = only(x)
    assert torch.is_tensor(out)
    empty, index = a(torch.zeros(0, 7))
    assert empty.shape == (1, 7) and index.numel() == 0 and a.active_bucket == 0


def test_member_lists_follow_the_index_tensor():
    torch.manual_seed(5)
    c = Compressgnn_Cluster(7, 4)
    x = torch.randn(30, 7)
    _, index = c(x)
    groups = c.active_bucket + 1
    m = cc.members_of(index, groups)
    assert m is not None and m[1].numel() == 30
    assert cc.members_of(index.clone(), groups) is None      # another tensor: nothing recorded
    assert cc.members_of(index, groups + 1) is None          # other number of groups
    index.add_(0)                                            # modified in place: not served
    assert cc.members_of(index, groups) is None
