"""compressgnn_sample: neighbour sampling over a compressed graph, on the GPU.

The reference builds a CPU module of this name from src/sample (function.cpp:7-9) with two
functions, neighbor_sample_cg_sim and neighbor_sample_ori_impl; both are here with the same
positional arguments and the same results -- (samples, rows, cols): the sampled vertices in
the order they were first met, and for every sampled edge the position of its endpoint among
them -- computed by HIP kernels on GPU tensors (CPU tensors raise).

Differences a caller can observe: the tensors live on the GPU; the random positions come from
a counter-based generator keyed by `seed` (an extra keyword, default 0; the same seed gives the
same sample whatever the scheduling) instead of torch's global CPU generator; where the
reference throws std::out_of_range (IndexError in Python) this raises IndexError as well.

sample_compress_graph(graph, ...) takes a CompressGraph (loader/compress_graph.py) directly.
"""
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.append(_HERE)

from compressgnn_runtime import neighbor_sample_cg_sim, neighbor_sample_ori_impl  # noqa: E402,F401


def sample_compress_graph(graph, input_node, num_neighbors, seed=0):
    """neighbor_sample_cg_sim on the blocks of a CompressGraph that lives on a GPU: the
    in-neighbours of the input vertices, `num_neighbors[l]` per vertex in layer l (all of them
    where a vertex has no more)."""
    held = getattr(graph, "_sampler_blocks", None)
    if held is None or held[0] != graph.device:
        # device copies of the int64 blocks for the sampler alone (the blocks themselves may rest
        # on the host once a propagation plan is built)
        v2v, v2r, r2v = graph.v2v_graph.csr(), graph.v2r_graph.csr(), graph.r2v_graph.csr()
        levels = [g.csr() for g in graph.r2r_graph]
        held = (graph.device, (v2v[0], v2v[1], v2r[0], v2r[1], r2v[0], r2v[1], [l[0] for l in levels],
                               [l[1] for l in levels], graph.vertex_degree, graph.rule_degree))
        graph._sampler_blocks = held
    return neighbor_sample_cg_sim(*held[1], input_node, list(num_neighbors), seed)
