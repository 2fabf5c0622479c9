"""Mean representatives with refreshable LSH assignments.

Same classes, constructor arguments, cache/refresh policy and return contracts as the
reference's layer/CompressgnnCluster.py:28-187.  Only indices, cluster counts and the
clusters' member lists are cached; representatives are recomputed from the current
features on every call so that gradients reach the current upstream model.  Call
set_epoch with zero-based epochs when refresh_interval > 1.  Train and eval keep separate
assignments; cache_key must identify a graph and node ordering.

All arithmetic runs in the HIP kernels behind compressgnn_runtime; CPU tensors are
rejected by those operators.
"""
import math
import operator
import weakref

import _paths  # noqa: F401
import torch
from torch.autograd.function import once_differentiable

import compressgnn_runtime as _native

# Member lists (offsets, perm, sorted_id) recorded for index tensors handed out by this
# module, keyed by the identity of the index tensor.  Compressgnn_Reconstruct looks its
# index argument up here so that the per-cluster gradient sum does not have to sort the
# ids again.  Entries vanish with their tensor; a tensor modified in place after it was
# recorded is not served.
_MEMBERS = {}


def _remember(index, members):
    key = id(index)

    def _drop(_ref, key=key):
        _MEMBERS.pop(key, None)

    _MEMBERS[key] = (weakref.ref(index, _drop), index._version, members)


def members_of(index, groups):
    """Recorded member lists for this very index tensor, or None."""
    entry = _MEMBERS.get(id(index))
    if entry is None:
        return None
    ref, version, members = entry
    if ref() is not index or index._version != version or members[0].numel() != groups + 1:
        return None
    return members


def _members(index, counts):
    members = members_of(index, counts.numel())
    if members is None:
        members = _native.cluster_members(index, counts.numel())
        _remember(index, members)
    return members


def _mean_forward(x, index, counts):
    """reference layer/CompressgnnCluster.py:16-19"""
    x = x.contiguous()
    if x.numel() == 0:
        return x.new_zeros((counts.numel(), x.size(1)))
    return _native.cluster_mean(x, index, counts, _members(index, counts))


def _mean_backward(grad, index, counts):
    """reference layer/CompressgnnCluster.py:22-25"""
    return _native.cluster_mean_backward(grad.contiguous(), index, counts, members_of(index, counts.numel()))


class _Mean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, index, counts):
        ctx.save_for_backward(index, counts)
        return _mean_forward(x, index, counts)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        index, counts = ctx.saved_tensors
        return _mean_backward(grad, index, counts), None, None


def _assign(input, planes, bits, workspace=None):
    """reference layer/CompressgnnCluster.py:41-50 (GPU branch).  One call yields the
    assignment and its member lists (the rows are grouped by a sort of their codes); the
    lists are recorded for the index tensor.  The bucket workspace of the reference's
    operator is not needed by this path."""
    with torch.no_grad():
        index, counts, active, members = _native.cluster_assign_members(input.contiguous(), planes.contiguous(), bits)
        _remember(index, tuple(members))
        return index, counts, active


class Compressgnn_Cluster_Function(torch.autograd.Function):
    """Compatibility entry point; fixed-assignment mean gradients, no cache."""
    @staticmethod
    def forward(ctx, input, random_vectors, param_H, is_training):
        index, counts, active = _assign(input, random_vectors, param_H)
        ctx.save_for_backward(index, counts)
        ctx.mark_non_differentiable(index)
        return _mean_forward(input, index, counts), index, active

    @staticmethod
    @once_differentiable
    def backward(ctx, grad, _index_grad, _active_grad):
        index, counts = ctx.saved_tensors
        return _mean_backward(grad, index, counts), None, None, None


class Compressgnn_Cluster(torch.nn.Module):
    """Reusable LSH indices; q is measured in epochs, never in forward calls.

    refresh_interval=1 refreshes on every epoch.  For q>1, call set_epoch(e), or pass
    epoch=e to forward.  A cache-disabled call always refreshes.  The legacy index_cache
    argument is accepted; both values cache indices only, never detached features.
    Constructor training=False retains the tensor-only return contract; training=True
    returns (representatives, index) in both train() and eval().  Module mode controls
    separate cache namespaces.
    """
    def __init__(self, in_feature, param_H, training=True, device=None, dtype=None,
                 cache=True, index_cache=False, refresh_interval=1,
                 refresh_policy='fixed', q_min=1, q_max=10, tau_loss=None):
        super().__init__()
        self.in_feature = operator.index(in_feature)
        self.param_H = operator.index(param_H)
        if self.in_feature < 0 or not 0 <= self.param_H <= 30:
            raise ValueError('Expected nonnegative feature width and 0 <= param_H <= 30')
        self.refresh_interval = operator.index(refresh_interval)
        self.q_min, self.q_max = operator.index(q_min), operator.index(q_max)
        if self.refresh_interval < 1 or not 1 <= self.q_min <= self.q_max:
            raise ValueError('Refresh intervals must be positive integers, q_min <= q_max')
        if refresh_policy not in ('fixed', 'loss'):
            raise ValueError('refresh_policy must be fixed or loss')
        if refresh_policy == 'loss' and (tau_loss is None or not math.isfinite(tau_loss) or tau_loss <= 0):
            raise ValueError('Loss policy requires a finite positive tau_loss')
        self.refresh_policy, self.tau_loss = refresh_policy, tau_loss
        self.cache, self.index_cache = bool(cache), bool(index_cache)
        self.is_training = bool(training)  # Legacy return contract, not cache mode.
        self.register_buffer('random_vectors', torch.randn(self.in_feature, self.param_H,
                                                           device=device, dtype=dtype))
        self._epoch = None
        self._previous_loss = None
        self._last_loss_epoch = None
        self.current_interval = self.refresh_interval if refresh_policy == 'fixed' else self.q_min
        self._states, self._workspaces = {}, {}
        self.vertex_index = self.active_bucket = None
        self.last_refreshed = False
        self.refresh_count = 0
        self.train(training)

    def set_epoch(self, epoch, loss=None):
        """Set zero-based epoch; loss is the previous completed training loss."""
        epoch = operator.index(epoch)
        if epoch < 0:
            raise ValueError('epoch must be nonnegative')
        if self._epoch is not None and epoch < self._epoch:
            self.reset_cache()
            self._previous_loss = self._last_loss_epoch = None
            self.current_interval = self.refresh_interval if self.refresh_policy == 'fixed' else self.q_min
        self._epoch = epoch
        if loss is not None and self.refresh_policy == 'loss' and epoch != self._last_loss_epoch:
            if torch.is_tensor(loss):
                raise TypeError('Pass a host loss value; do not hide a GPU synchronization in set_epoch')
            loss = float(loss)
            if not math.isfinite(loss):
                raise ValueError('loss must be finite')
            if self._previous_loss is not None:
                raw = self.q_min + (self.q_max - self.q_min) * math.exp(-abs(loss - self._previous_loss) / self.tau_loss)
                self.current_interval = min(self.q_max, max(self.q_min, int(math.floor(raw + .5))))
            self._previous_loss, self._last_loss_epoch = loss, epoch
        return self

    def reset_cache(self):
        self._states.clear()
        self.vertex_index = self.active_bucket = None
        self.last_refreshed = False

    def _apply(self, fn, *args, **kwargs):
        self.reset_cache()
        self._workspaces.clear()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self.reset_cache()
        self._previous_loss = self._last_loss_epoch = None
        self._epoch = None
        self.current_interval = self.refresh_interval if self.refresh_policy == 'fixed' else self.q_min
        return super()._load_from_state_dict(*args, **kwargs)

    def forward(self, input, epoch=None, cache_key=None, force_refresh=False):
        if input.dim() != 2 or input.size(1) != self.in_feature:
            raise ValueError('Expected [nodes, in_feature] input')
        if input.device != self.random_vectors.device or input.dtype != self.random_vectors.dtype:
            raise ValueError('Move the module to the input device and dtype before use')
        if input.dtype not in (torch.float32, torch.float64):
            raise ValueError('Only float32 and float64 are supported')
        if epoch is not None:
            self.set_epoch(epoch)
        if self.cache and self._epoch is None and (self.refresh_interval > 1 or self.refresh_policy == 'loss'):
            raise ValueError('Cross-epoch reuse requires set_epoch(epoch) or forward(epoch=epoch)')
        # Assignments are kept per mode, device and stream.
        stream = torch.cuda.current_stream(input.device).cuda_stream if input.is_cuda else None
        slot = (self.training, input.device, stream)
        signature = (tuple(input.shape), input.dtype, cache_key, self.random_vectors.data_ptr(),
                     self.random_vectors._version)
        state = self._states.get(slot)
        refresh = (not self.cache or force_refresh or self._epoch is None or state is None or
                   state['signature'] != signature or self._epoch - state['epoch'] >= self.current_interval)
        if refresh:
            if not input.size(0):
                index = torch.empty(0, device=input.device, dtype=torch.int64)
                counts = torch.zeros(1, device=input.device, dtype=torch.int32)
                active = 0
            else:
                # the member lists of the new assignment come with it and are reused by
                # every mean and reconstruct-gradient until the next refresh
                index, counts, active = _assign(input, self.random_vectors, self.param_H)
            state = dict(index=index, counts=counts, active=active, signature=signature, epoch=self._epoch)
            if self.cache and self._epoch is not None:
                self._states[slot] = state
            self.refresh_count += 1
        self.last_refreshed = refresh
        self.vertex_index, self.active_bucket = state['index'], state['active']
        output = _Mean.apply(input, state['index'], state['counts'])
        return (output, state['index']) if self.is_training else output
