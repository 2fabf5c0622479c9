"""The batch compressor on the GPU (module compressgnn_batch_cuda): its output is held to the
contract the reference's tests pin at the compressor boundary -- int32 arrays, children below the
rule's id, every vertex row expanding to exactly the input row in order
(tests/test_batch_compression.py:15-36,52-55, tests/test_offline_compression.py:7-25), checked by
a numpy expansion that shares no code with the product -- and, beside that, to the arrays of the
host compressor (tests/test_batch_compression.py:52-59 asks that of the two backends), on the
reference's grid of row shapes and on the graphs of the benchmark configurations."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd"))
sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd", "loader"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

pytestmark = pytest.mark.gpu


def both(v, e, rounds, freq):
    import compressgnn_batch_cuda as gpu
    from compressgnn_amd import compressgnn_offline as off
    want = off.compress_csr_batch(v, e, 4, rounds, freq)
    from util import assert_compression_contract
    got = gpu.compress_csr_batch(v, e, rounds=rounds, min_pair_frequency=freq)
    assert_compression_contract(v, e, got)
    assert got[2] == want[2] and got[3] == want[3]
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    return got


def test_gpu_compressor_matches_host_on_row_shapes():
    import compressgnn_batch_cuda as gpu
    assert gpu.is_available()
    rng = np.random.default_rng(73)
    for n in [1, 2, 17, 128, 512]:
        fixtures = [
            [[] for _ in range(n)],
            [[i] for i in range(n)],
            [list(range(min(n, 16))) for _ in range(n)],
            [sorted(rng.choice(n, size=min(n, 20), replace=False).tolist()) for _ in range(n)],
            [sorted(rng.integers(n, size=8).tolist()) for _ in range(n)],
            [rng.integers(min(n, 6), size=int(rng.integers(0, 40))).tolist() for _ in range(n)],  # long stretches
        ]
        for rows in fixtures:
            v = np.array([0] + list(np.cumsum([len(x) for x in rows])), dtype=np.int32)
            e = np.array([j for row in rows for j in row], dtype=np.int32)
            for freq in [3, 4, 16]:
                both(v, e, 12, freq)
    # [0] * 50: one stretch of 49 matched positions, taken at every other one
    v = np.array([0, 50, 100, 150], np.int64)
    e = np.zeros(150, np.int64)
    got = both(v, e, 12, 3)
    assert got[3] > 0
    # 64 identical rows share everything
    v = np.arange(65, dtype=np.int64) * 32
    e = np.tile(np.arange(32, dtype=np.int64), 64)
    got = both(v, e, 12, 16)
    assert got[3] > 0 and len(got[1]) < len(e) // 4
    both(v, e, 1, 16)
    both(v, e, 3, 16)
    assert gpu.compress_csr_batch(np.zeros(0, np.int64), np.zeros(0, np.int64))[2:] == (0, 0)


@pytest.mark.parametrize("graph", ["chung_lu", "copy_model", "copy_model_large"])
def test_gpu_compressor_matches_host_on_graphs(graph):
    from compressgnn_amd import compressgnn_offline as off
    if graph == "chung_lu":
        v, e = off.gen_chung_lu(2708, 10500, 2.5, 3)
        freq = 3
    elif graph == "copy_model":
        v, e = off.gen_copy_model(20000, 9.8, 0.7, 5)
        freq = 8
    else:
        v, e = off.gen_copy_model(325557, 9.8, 0.7, 1)
        freq = 16
    v, e = off.add_self_loop_csr(v, e)
    got = both(v, e, 12, freq)
    assert got[3] > 0


def test_gpu_compressor_rejects_bad_input_and_is_the_loaders_choice():
    import compressgnn_batch_cuda as gpu
    import compression_backend
    for freq in [-1, 0, 1, 2]:
        with pytest.raises(ValueError):
            gpu.compress_csr_batch(np.array([0, 0], np.int32), np.array([], np.int32), min_pair_frequency=freq)
    with pytest.raises(ValueError):
        gpu.compress_csr_batch(np.array([0, 1], np.int64), np.array([2 ** 32], np.uint64))
    with pytest.raises(ValueError):
        gpu.compress_csr_batch(np.array([0, 1]), np.array([0.5]))
    with pytest.raises(ValueError):  # column outside [0, V)
        gpu.compress_csr_batch(np.array([0, 1], np.int64), np.array([7], np.int64))
    with pytest.raises(ValueError):  # row starts that do not end at E
        gpu.compress_csr_batch(np.array([0, 3], np.int64), np.array([0], np.int64))
    assert compression_backend.resolve_backend("auto") == "cuda"
    assert compression_backend.resolve_backend("cuda") == "cuda"
    v = np.arange(65, dtype=np.int64) * 32
    e = np.tile(np.arange(32, dtype=np.int64), 64) % 64
    a = compression_backend.compress_graph_csr(v, e, 16, backend="cuda")
    b = compression_backend.compress_graph_csr(v, e, 16, backend="cpu")
    assert all(np.array_equal(x, y) for x, y in zip(a[:2], b[:2])) and a[2:] == b[2:]


def test_loader_gives_the_same_dataset_on_either_backend():
    """CompressgnnData with the work on the GPU (rule merger and the by-column form of the
    compressed matrix) holds the same blocks, weights and degrees as with everything on the host."""
    sys.path.insert(0, os.path.join(ROOT, "compressgnn_amd", "layer"))
    from compressgnn_amd import compressgnn_offline as off
    from CompressgnnData import CompressgnnData
    v, e = off.gen_copy_model(20000, 9.8, 0.7, 11)
    V = len(v) - 1
    m = np.ones(V, bool)
    both = [CompressgnnData(np.zeros((V, 1), np.float32), (v, e), np.zeros(V, np.int64), m, m, m, graph_type="csr",
                            min_pair_frequency=4, compression_backend=backend, verbose=False) for backend in ("cuda", "cpu")]
    a, b = (d.edge_index for d in both)
    assert (both[0].vertex_cnt, both[0].rule_cnt, both[0].edge_cnt, a.step) == (both[1].vertex_cnt, both[1].rule_cnt, both[1].edge_cnt, b.step)
    assert both[0].rule_cnt > 0
    for x, y in zip(a.blocks(), b.blocks()):
        for p, q in zip(x.csr(), y.csr()):
            assert p.dtype == q.dtype and np.array_equal(p.cpu().numpy(), q.cpu().numpy())
    assert np.array_equal(a.vertex_degree.numpy(), b.vertex_degree.numpy())
    assert np.array_equal(a.rule_degree.numpy(), b.rule_degree.numpy())
