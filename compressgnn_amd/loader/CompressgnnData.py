"""CompressgnnData: from raw arrays to the compressed, normalised, partitioned graph.

The constructor arguments, the fields it leaves on the object (x, y, the three masks,
vertex_cnt, rule_cnt, edge_cnt, feature_dim, graph_type, step, edge_index, edge_weight for
"coo", and the compression settings), to() and the text of __repr__ are those of the
reference's loader/CompressgnnData.py:60-201.  graph_type="csr" ends in a CompressGraph,
graph_type="coo" in one [2, E_k] edge tensor and one weight vector per phase.

Pipeline (the reference's order): self loops -> normalised degrees of the uncompressed
graph -> batch compression -> saving filter -> depth filter -> weights of the compressed
edges -> partition ("csr") or phase masks ("coo").
"""
import copy

import _paths  # noqa: F401
import numpy as np
import torch
import torch.utils.data

import compressgnn_offline as offline
from compress_graph import CompressGraph
from compression_backend import compress_graph_csr, resolve_backend


def _size(vlist, elist):
    return int(vlist.shape[0]) + int(elist.shape[0])


def compress(vlist, elist, threshold, max_depth, min_edge, min_pair_frequency=16,
             compression_backend='auto', compression_threads=4, compression_rounds=12, verbose=True):
    """Batch compression, saving filter, depth filter (loader/CompressgnnData.py:26-55 of the
    reference).  Returns (vlist, elist, vertex_cnt, rule_cnt) of the compressed graph; with
    verbose, prints the size ratio after every stage."""
    backend = resolve_backend(compression_backend)
    original = _size(vlist, elist)
    stages = (
        ('batch compression (%s)' % backend,
         lambda g: compress_graph_csr(vlist, elist, min_pair_frequency, backend, compression_threads,
                                      compression_rounds)),
        ('saving filter', lambda g: offline.filter_csr(g[0], g[1], g[2], g[3], threshold)),
        ('depth filter', lambda g: offline.depth_filter_csr(g[0], g[1], g[2], g[3], max_depth, min_edge)),
    )
    graph = None
    for name, run in stages:
        graph = run(graph)
        if verbose:
            now = _size(graph[0], graph[1])
            print('%-28s size %d -> %d, ratio %.4f, %d rules' % (name, original, now, original / now, graph[3]))
    return graph


class CompressgnnData():
    def __init__(self, x, edge_index, y,
                 train_mask, vaild_mask, test_mask,
                 add_self_loop: bool = True, normalize: bool = True,
                 graph_type: str = "coo",
                 max_depth: int = 3,
                 min_edge: int = 1000000,
                 threshold: int = 16,
                 homo: bool = False,
                 min_pair_frequency: int = 16,
                 compression_backend: str = "auto",
                 compression_threads: int = 4,
                 compression_rounds: int = 12,
                 verbose: bool = False):
        if graph_type not in ("coo", "csr"):
            raise ValueError('graph_type must be "coo" or "csr"')
        self.x = torch.as_tensor(np.asarray(x).astype(np.float32))
        self.y = torch.as_tensor(np.array(y))
        for name, mask in (("train_mask", train_mask), ("vaild_mask", vaild_mask), ("test_mask", test_mask)):
            setattr(self, name, torch.as_tensor(mask))
        self.vertex_cnt, self.feature_dim = self.x.size()[0], self.x.size()[1]
        self.graph_type = graph_type
        self.min_pair_frequency = min_pair_frequency
        self.compression_backend = resolve_backend(compression_backend)
        self.compression_threads = compression_threads
        self.compression_rounds = compression_rounds
        self._settings = dict(threshold=threshold, max_depth=max_depth, min_edge=min_edge,
                              min_pair_frequency=min_pair_frequency, compression_backend=self.compression_backend,
                              compression_threads=compression_threads, compression_rounds=compression_rounds,
                              verbose=verbose)
        first = np.asarray(edge_index[0]).astype(np.int64)
        second = np.asarray(edge_index[1]).astype(np.int64)
        if graph_type == "csr":
            self._from_csr(first, second, add_self_loop, normalize)
        else:
            self._from_edges(first, second, add_self_loop, normalize, verbose)

    def _compressed(self, vlist, elist):
        vlist, elist, self.vertex_cnt, self.rule_cnt = compress(vlist, elist, **self._settings)
        self.edge_cnt = elist.shape[0]
        return vlist.astype(np.int64), elist.astype(np.int64)

    # graph_type="csr": (vlist, elist) -> CompressGraph  (loader/CompressgnnData.py:140-181)
    def _from_csr(self, vlist, elist, add_self_loop, normalize):
        if add_self_loop:
            vlist, elist = offline.add_self_loop_csr(vlist, elist)
        degree = offline.get_norm_degree(elist, self.vertex_cnt) if normalize else None
        vlist, elist = self._compressed(vlist, elist)
        if normalize:
            weight = offline.gcn_norm_csr_compress(vlist, elist, degree, self.vertex_cnt, self.rule_cnt)
        else:
            weight = np.ones(self.edge_cnt, dtype=np.float32)
        # `step` is the phase count the reference reports for this form (its
        # gen_mask_vertex(..., "csc"), :177-179); the kernels go by CompressGraph.step
        self.step = offline.gen_vertex_order_csc(vlist, elist, self.vertex_cnt, self.rule_cnt)[1]
        nodes = self.vertex_cnt + self.rule_cnt
        colptr, row, value = self._by_column(vlist, elist, weight, nodes)
        self.edge_index = CompressGraph(colptr, row, value, self.vertex_cnt)

    def _by_column(self, vlist, elist, weight, nodes):
        """The compressed matrix by column (SparseTensor.csc() of the reference, :180): on the GPU
        when the loader already works there (compression_backend 'cuda'), the same arrays bit for
        bit as the host routine; a graph that does not fit the device beside what is there goes to
        the host routine."""
        if self.compression_backend == 'cuda':
            import compressgnn_runtime as rt
            dev = torch.device('cuda', torch.cuda.current_device())
            try:
                parts = rt.csr_transpose(torch.from_numpy(vlist).to(dev), torch.from_numpy(elist).to(dev),
                                         torch.from_numpy(weight).to(dev), nodes)
                return tuple(p.cpu().numpy() for p in parts)
            except torch.cuda.OutOfMemoryError:
                pass
        return offline.csr_transpose(vlist, elist, weight, nodes)

    # graph_type="coo": (src, dst) -> edge and weight tensors per phase  (:86-139)
    def _from_edges(self, src, dst, add_self_loop, normalize, verbose):
        if add_self_loop:
            src, dst = offline.add_self_loop_coo(src, dst, self.vertex_cnt)
        degree = offline.get_norm_degree(dst, self.vertex_cnt) if normalize else None
        vlist, elist = self._compressed(*offline.coo2csr(src, dst, self.vertex_cnt))
        src, dst = offline.csr2coo(vlist, elist)
        if normalize:
            weight = offline.gcn_norm_coo_compress(src, dst, degree, self.vertex_cnt, self.rule_cnt)
        else:
            weight = np.ones(self.edge_cnt, dtype=np.float32)
        phase_masks, self.step = offline.gen_mask_edge(src, dst, self.vertex_cnt, self.rule_cnt)
        if verbose:
            print("phases: %d" % self.step)
        edges = torch.from_numpy(np.vstack((src, dst)))
        weights = torch.from_numpy(weight)
        self.edge_index, self.edge_weight = [], []
        for k in range(self.step):
            keep = torch.from_numpy(phase_masks[k])
            self.edge_index.append(edges[:, keep].contiguous())
            self.edge_weight.append(weights[keep])

    def __repr__(self):
        shown = (self.vertex_cnt, self.rule_cnt, self.edge_cnt, self.step, self.graph_type)
        return 'CompressgnnData(vertex_cnt:"%s", rule_cnt:"%s", edge_cnt:"%s", step:"%s", graph_type:"%s")' % shown

    def to(self, device):
        for name in ("x", "y", "train_mask", "vaild_mask", "test_mask"):
            setattr(self, name, getattr(self, name).to(device))
        if self.graph_type == "csr":
            self.edge_index = self.edge_index.to(device)
        else:
            self.edge_index = [e.to(device) for e in self.edge_index]
            self.edge_weight = [w.to(device) for w in self.edge_weight]
        return self


class CompressgnnBatchData():
    """A sequence of prepared datasets stored in one file (loader/CompressgnnData.py:203-209 of
    the reference): `torch.save([data_0, data_1, ...], path)` of CompressgnnData objects made by
    this library.  The file holds pickled objects, so it is opened with the unpickler: load only
    files that this library wrote."""

    def __init__(self, path):
        self.data = torch.load(path, weights_only=False)
        self.len = len(self.data)

    def __len__(self):
        return self.len


class CompressgnnDataLoader(torch.utils.data.DataLoader):
    """Hands out the datasets of a CompressgnnBatchData one per step
    (loader/CompressgnnData.py:212-222): the loader walks the positions, and a step is a shallow
    copy of the dataset at the first position of its batch, as in the reference."""

    def __init__(self, data, **kwargs):
        self.data = data
        super().__init__(range(len(data)), collate_fn=self.__collate__, **kwargs)

    def __collate__(self, batch):
        return copy.copy(self.data.data[int(batch[0])])
