"""Cluster representatives over refreshable LSH assignments.

Public surface of the reference's layer/CompressgnnCluster.py:28-187: the module
Compressgnn_Cluster (constructor arguments, set_epoch / reset_cache / forward, the
counters refresh_count, last_refreshed, vertex_index, active_bucket, current_interval)
and the function-style entry point Compressgnn_Cluster_Function.

What is kept between calls is the assignment only: ids, cluster sizes and the clusters'
member lists.  The representatives themselves are recomputed from the features of the
call, so their gradient always reaches the model that produced those features.  Epochs
are zero based; an interval of q epochs means "assign again once q epochs have passed
since the last assignment".  train() and eval() keep separate assignments, and so do
different devices and streams.

Every operator here is a HIP kernel behind compressgnn_runtime; there is no CPU path.
"""
import math
import operator
import weakref

import _paths  # noqa: F401
import torch
from torch.autograd.function import once_differentiable

import compressgnn_runtime as _native


# ----------------------------------------------------------------- member lists --
class _MemberLists:
    """Member lists (offsets, perm, sorted_id) of the index tensors this module hands
    out, looked up by tensor identity.  Compressgnn_Reconstruct asks here so that its
    per-cluster gradient sum needs no second sort of the ids.  An entry goes away with
    its tensor, and a tensor that was written to after it was recorded is not served."""

    def __init__(self):
        self._by_id = {}

    def record(self, index, lists):
        ident = id(index)
        forget = lambda _gone, ident=ident: self._by_id.pop(ident, None)
        self._by_id[ident] = (weakref.ref(index, forget), index._version, tuple(lists))

    def lookup(self, index, groups):
        found = self._by_id.get(id(index))
        if found is None:
            return None
        alive, version, lists = found
        stale = alive() is not index or index._version != version or lists[0].numel() != groups + 1
        return None if stale else lists

    def ensure(self, index, groups):
        lists = self.lookup(index, groups)
        if lists is None:
            lists = tuple(_native.cluster_members(index, groups))
            self.record(index, lists)
        return lists


_LISTS = _MemberLists()


def members_of(index, groups):
    """Recorded member lists of exactly this index tensor, or None."""
    return _LISTS.lookup(index, groups)


# ------------------------------------------------------------ operators + autograd --
def _assign(input, planes, bits, workspace=None):
    """Hash, dense ids, cluster sizes and member lists in one native call (the rows are
    grouped by sorting their codes).  Takes the place of the workspace / assign pair of
    layer/CompressgnnCluster.py:41-50; a workspace argument is accepted and unused."""
    with torch.no_grad():
        index, counts, active, lists = _native.cluster_assign_members(input.contiguous(), planes.contiguous(), bits)
    _LISTS.record(index, lists)
    return index, counts, active


def _representatives(x, index, counts):
    # sum of the members / max(size, 1): scatter_mean of layer/CompressgnnCluster.py:16-19
    x = x.contiguous()
    groups = counts.numel()
    if x.numel() == 0:
        return x.new_zeros((groups, x.size(1)))
    return _native.cluster_mean(x, index, counts, _LISTS.ensure(index, groups))


def _spread(grad, index, counts):
    # every member receives its cluster's gradient / max(size, 1) (layer/CompressgnnCluster.py:22-25)
    return _native.cluster_mean_backward(grad.contiguous(), index, counts, members_of(index, counts.numel()))


class _Mean(torch.autograd.Function):
    """Representatives of a fixed assignment; first-order gradient with respect to x."""

    @staticmethod
    def forward(ctx, x, index, counts):
        ctx.save_for_backward(index, counts)
        return _representatives(x, index, counts)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        return (_spread(grad, *ctx.saved_tensors), None, None)


class Compressgnn_Cluster_Function(torch.autograd.Function):
    """apply(input, random_vectors, param_H, is_training) -> (representatives, index,
    active): assigns on every call, keeps nothing."""

    @staticmethod
    def forward(ctx, input, random_vectors, param_H, is_training):
        index, counts, active = _assign(input, random_vectors, param_H)
        ctx.mark_non_differentiable(index)
        ctx.save_for_backward(index, counts)
        return _representatives(input, index, counts), index, active

    @staticmethod
    @once_differentiable
    def backward(ctx, grad, *_unused):
        return (_spread(grad, *ctx.saved_tensors), None, None, None)


# ------------------------------------------------------------------- the schedule --
def _whole(value, what, low=None, high=None):
    number = operator.index(value)
    if (low is not None and number < low) or (high is not None and number > high):
        raise ValueError('%s is out of range: %r' % (what, value))
    return number


class _Schedule:
    """Which epoch it is and how many epochs an assignment lasts.  'fixed': always
    `interval`.  'loss': q_min + (q_max - q_min) * exp(-|loss - previous loss| / tau),
    rounded half up and kept inside [q_min, q_max] (layer/CompressgnnCluster.py:126-128);
    q_min until two losses have been seen."""

    def __init__(self, policy, interval, q_min, q_max, tau):
        self.policy, self.fixed, self.q_min, self.q_max, self.tau = policy, interval, q_min, q_max, tau
        self.forget()

    def forget(self):
        self.epoch = None
        self.loss = None
        self.loss_epoch = None
        self.interval = self.fixed if self.policy == 'fixed' else self.q_min

    def needs_epoch(self):
        return self.epoch is None and (self.policy == 'loss' or self.fixed > 1)

    def rewinds(self, epoch):
        return self.epoch is not None and epoch < self.epoch

    def advance(self, epoch, loss):
        if self.rewinds(epoch):
            self.forget()
        self.epoch = epoch
        if loss is None or self.policy != 'loss' or epoch == self.loss_epoch:
            return
        if torch.is_tensor(loss):
            raise TypeError('set_epoch takes the loss as a Python number: reading a tensor here would '
                            'synchronise with the device')
        loss = float(loss)
        if not math.isfinite(loss):
            raise ValueError('the loss passed to set_epoch is not finite')
        if self.loss is not None:
            q = self.q_min + (self.q_max - self.q_min) * math.exp(-abs(loss - self.loss) / self.tau)
            self.interval = max(self.q_min, min(self.q_max, int(math.floor(q + 0.5))))
        self.loss, self.loss_epoch = loss, epoch


class _Assignment:
    __slots__ = ('index', 'counts', 'active', 'signature', 'epoch')

    def __init__(self, index, counts, active, signature, epoch):
        self.index, self.counts, self.active, self.signature, self.epoch = index, counts, active, signature, epoch


# --------------------------------------------------------------------- the module --
class Compressgnn_Cluster(torch.nn.Module):
    """forward(input[N, in_feature]) -> representatives[C, in_feature], and the index
    tensor as well when the constructor's `training` is true (that flag only selects the
    return form; train()/eval() select which cached assignment is used).

    With cache=True an assignment is reused until `current_interval` epochs have passed,
    the input's shape, dtype or cache_key changes, the hash planes change, or
    force_refresh is given; the epoch comes from set_epoch(e) or forward(epoch=e) and is
    required when an assignment may outlive an epoch.  cache=False assigns on every call.
    index_cache is accepted for compatibility and changes nothing."""

    def __init__(self, in_feature, param_H, training=True, device=None, dtype=None,
                 cache=True, index_cache=False, refresh_interval=1,
                 refresh_policy='fixed', q_min=1, q_max=10, tau_loss=None):
        super().__init__()
        self.in_feature = _whole(in_feature, 'in_feature', low=0)
        self.param_H = _whole(param_H, 'param_H', low=0, high=30)
        self.refresh_interval = _whole(refresh_interval, 'refresh_interval', low=1)
        self.q_min = _whole(q_min, 'q_min', low=1)
        self.q_max = _whole(q_max, 'q_max', low=self.q_min)
        if refresh_policy == 'loss':
            if tau_loss is None or not (math.isfinite(tau_loss) and tau_loss > 0):
                raise ValueError("refresh_policy='loss' needs tau_loss > 0")
        elif refresh_policy != 'fixed':
            raise ValueError("refresh_policy is 'fixed' or 'loss'")
        self.refresh_policy = refresh_policy
        self.tau_loss = tau_loss
        self.cache = bool(cache)
        self.index_cache = bool(index_cache)
        self.is_training = bool(training)
        planes = torch.randn(self.in_feature, self.param_H, device=device, dtype=dtype)
        self.register_buffer('random_vectors', planes)
        self._schedule = _Schedule(refresh_policy, self.refresh_interval, self.q_min, self.q_max, tau_loss)
        self._assignments = {}
        self.refresh_count = 0
        self._clear_view()
        self.train(training)

    # what the last forward call used
    def _clear_view(self):
        self.vertex_index = None
        self.active_bucket = None
        self.last_refreshed = False

    @property
    def current_interval(self):
        return self._schedule.interval

    def set_epoch(self, epoch, loss=None):
        """Zero-based epoch about to run; with the loss policy, `loss` is the loss of the
        epoch that just finished.  Going back to an earlier epoch starts over."""
        epoch = _whole(epoch, 'epoch', low=0)
        if self._schedule.rewinds(epoch):
            self.reset_cache()
        self._schedule.advance(epoch, loss)
        return self

    def reset_cache(self):
        self._assignments.clear()
        self._clear_view()

    def _apply(self, fn, *args, **kwargs):
        # .to() / .double() / .cuda(): the hash planes move or change, assignments are void
        self.reset_cache()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self.reset_cache()
        self._schedule.forget()
        return super()._load_from_state_dict(*args, **kwargs)

    def _check_input(self, input):
        planes = self.random_vectors
        if input.dim() != 2 or input.size(1) != self.in_feature:
            raise ValueError('input must be [nodes, %d]' % self.in_feature)
        if input.device != planes.device or input.dtype != planes.dtype:
            raise ValueError('input and module differ in device or dtype (%s %s against %s %s)'
                             % (input.device, input.dtype, planes.device, planes.dtype))
        if input.dtype not in (torch.float32, torch.float64):
            raise ValueError('float32 or float64 features only')

    def _fresh(self, input, signature):
        if input.size(0) == 0:
            index = torch.empty(0, dtype=torch.int64, device=input.device)
            counts = torch.zeros(1, dtype=torch.int32, device=input.device)
            active = 0
        else:
            index, counts, active = _assign(input, self.random_vectors, self.param_H)
        self.refresh_count += 1
        return _Assignment(index, counts, active, signature, self._schedule.epoch)

    def forward(self, input, epoch=None, cache_key=None, force_refresh=False):
        self._check_input(input)
        if epoch is not None:
            self.set_epoch(epoch)
        schedule = self._schedule
        if self.cache and schedule.needs_epoch():
            raise ValueError('assignments that last more than one epoch need set_epoch(e) or forward(epoch=e)')
        planes = self.random_vectors
        stream = torch.cuda.current_stream(input.device).cuda_stream if input.is_cuda else None
        slot = (self.training, input.device, stream)
        signature = (tuple(input.shape), input.dtype, cache_key, planes.data_ptr(), planes._version)
        held = self._assignments.get(slot) if self.cache and not force_refresh and schedule.epoch is not None else None
        usable = (held is not None and held.signature == signature
                  and schedule.epoch - held.epoch < schedule.interval)
        if not usable:
            held = self._fresh(input, signature)
            if self.cache and schedule.epoch is not None:
                self._assignments[slot] = held
        self.last_refreshed = not usable
        self.vertex_index, self.active_bucket = held.index, held.active
        reps = _Mean.apply(input, held.index, held.counts)
        return (reps, held.index) if self.is_training else reps
