"""Which batch compressor runs: resolve_backend / compress_graph_csr with the interface of
the reference's loader/compression_backend.py:6-40.

Two compressors produce the same arrays: the host one (compressgnn_offline.compress_csr_batch)
and the GPU one (module compressgnn_batch_cuda, HIP kernels).  'auto' means the GPU one
whenever a GPU can be used, 'cuda' insists on it, 'cpu' on the host one.
"""
import _paths  # noqa: F401
import importlib
import operator

_CHOICES = ('auto', 'cpu', 'cuda')


def _gpu_compressor():
    """(module, None) when the GPU compressor can run, else (None, (reason, cause))."""
    try:
        module = importlib.import_module('compressgnn_batch_cuda')
    except ImportError as missing:
        return None, ('the GPU compressor (module compressgnn_batch_cuda) is not importable', missing)
    if module.is_available():
        return module, None
    return None, ('the GPU compressor was asked for, but no GPU is usable', None)


def resolve_backend(backend):
    """'cpu' or 'cuda' for any of 'auto', 'cpu', 'cuda'; raises when 'cuda' cannot be had."""
    if backend not in _CHOICES:
        raise ValueError("compression_backend is one of %s, not %r" % (", ".join(map(repr, _CHOICES)), backend))
    if backend == 'cpu':
        return 'cpu'
    module, problem = _gpu_compressor()
    if module is None and backend == 'cuda':
        raise RuntimeError(problem[0]) from problem[1]
    return 'cpu' if module is None else 'cuda'


def _at_least(value, least, what):
    number = operator.index(value)
    if number < least:
        raise ValueError('%s must be at least %d, got %r' % (what, least, value))
    return number


def compress_graph_csr(vlist, elist, min_pair_frequency=16, backend='auto', threads=4, rounds=12):
    """(vlist, elist, vertex_cnt, rule_cnt) of the compressed graph.  Failures of the chosen
    compressor are raised, never answered by trying the other one."""
    pair_frequency = operator.index(min_pair_frequency)
    workers = _at_least(threads, 1, 'compression_threads')
    passes = _at_least(rounds, 1, 'compression_rounds')
    where = resolve_backend(backend)
    _at_least(pair_frequency, 3, 'min_pair_frequency')
    if where == 'cpu':
        host = importlib.import_module('compressgnn_offline')
        return host.compress_csr_batch(vlist, elist, threads=workers, rounds=passes, min_pair_frequency=pair_frequency)
    device, _ = _gpu_compressor()
    return device.compress_csr_batch(vlist, elist, rounds=passes, min_pair_frequency=pair_frequency)
