"""CompressgnnData: builds the compressed, normalised, partitioned graph from raw
arrays.  Same constructor, fields, to() and __repr__ as the reference's
loader/CompressgnnData.py:60-201: graph_type="csr" yields a CompressGraph, graph_type="coo"
per-phase edge lists and weights."""
import _paths  # noqa: F401
import numpy as np
import torch

from compressgnn_offline import (add_self_loop_coo, add_self_loop_csr, coo2csr, csr2coo, csr_transpose,
                                 depth_filter_csr, filter_csr, gcn_norm_coo_compress, gcn_norm_csr_compress,
                                 gen_mask_edge, gen_vertex_order_csc, get_norm_degree)
from compress_graph import CompressGraph
from compression_backend import compress_graph_csr, resolve_backend


def compress(vlist, elist, threshold, max_depth, min_edge, min_pair_frequency=16,
             compression_backend='auto', compression_threads=4, compression_rounds=12, verbose=True):
    """Batch compression, then the saving filter, then the depth filter
    (reference loader/CompressgnnData.py:26-55)."""
    say = print if verbose else (lambda *a, **k: None)
    selected = resolve_backend(compression_backend)
    say('Compression backend: {}'.format(selected))
    before = vlist.shape[0] + elist.shape[0]
    result = compress_graph_csr(vlist, elist, min_pair_frequency, selected, compression_threads, compression_rounds)
    new_vlist, new_elist, new_vertex_cnt, new_rule_cnt = result
    say("compression ratio: {} / {} = {:.4f}".format(before, new_vlist.shape[0] + new_elist.shape[0],
                                                     before / (new_vlist.shape[0] + new_elist.shape[0])))
    new_vlist, new_elist, new_vertex_cnt, new_rule_cnt = filter_csr(
        new_vlist, new_elist, new_vertex_cnt, new_rule_cnt, threshold)
    say("After filter compression ratio: {} / {} = {:.4f}".format(
        before, new_vlist.shape[0] + new_elist.shape[0], before / (new_vlist.shape[0] + new_elist.shape[0])))
    new_vlist, new_elist, new_vertex_cnt, new_rule_cnt = depth_filter_csr(
        new_vlist, new_elist, new_vertex_cnt, new_rule_cnt, max_depth, min_edge)
    say("After depth filter compression ratio: {} / {} = {:.4f}".format(
        before, new_vlist.shape[0] + new_elist.shape[0], before / (new_vlist.shape[0] + new_elist.shape[0])))
    return new_vlist, new_elist, new_vertex_cnt, new_rule_cnt


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
        x = np.asarray(x).astype(np.float32)
        self.x = torch.as_tensor(x)
        self.y = torch.as_tensor(np.array(y))
        self.train_mask = torch.as_tensor(train_mask)
        self.vaild_mask = torch.as_tensor(vaild_mask)
        self.test_mask = torch.as_tensor(test_mask)
        self.vertex_cnt = self.x.size()[0]
        self.feature_dim = self.x.size()[1]
        self.graph_type = graph_type
        self.min_pair_frequency = min_pair_frequency
        self.compression_backend = resolve_backend(compression_backend)
        self.compression_threads = compression_threads
        self.compression_rounds = compression_rounds
        if self.graph_type == "csr":
            vlist = np.asarray(edge_index[0]).astype(np.int64)
            elist = np.asarray(edge_index[1]).astype(np.int64)
            if add_self_loop:
                vlist, elist = add_self_loop_csr(vlist, elist)
            if normalize:
                norm_degree = get_norm_degree(elist, self.vertex_cnt)
            new_vlist, new_elist, vertex_cnt, rule_cnt = compress(
                vlist, elist, threshold, max_depth, min_edge, min_pair_frequency,
                self.compression_backend, compression_threads, compression_rounds, verbose)
            self.vertex_cnt = vertex_cnt
            self.rule_cnt = rule_cnt
            self.edge_cnt = new_elist.shape[0]
            new_vlist = new_vlist.astype(np.int64)
            new_elist = new_elist.astype(np.int64)
            if normalize:
                edge_weight = gcn_norm_csr_compress(new_vlist, new_elist, norm_degree, self.vertex_cnt, self.rule_cnt)
            else:
                edge_weight = np.ones(self.edge_cnt, dtype=np.float32)
            # the phase count the reference reports (gen_mask_vertex(..., "csc"),
            # loader/CompressgnnData.py:177-179); the kernels use CompressGraph.step instead
            _, self.step = gen_vertex_order_csc(new_vlist, new_elist, self.vertex_cnt, self.rule_cnt)
            total = vertex_cnt + rule_cnt
            colptr, row, value = csr_transpose(new_vlist, new_elist, edge_weight, total)
            self.edge_index = CompressGraph(colptr, row, value, self.vertex_cnt)
        elif self.graph_type == "coo":
            # reference loader/CompressgnnData.py:86-139: edges sorted by source
            src = np.asarray(edge_index[0]).astype(np.int64)
            dst = np.asarray(edge_index[1]).astype(np.int64)
            if add_self_loop:
                src, dst = add_self_loop_coo(src, dst, self.vertex_cnt)
            if normalize:
                norm_degree = get_norm_degree(dst, self.vertex_cnt)
            vlist, elist = coo2csr(src, dst, self.vertex_cnt)
            new_vlist, new_elist, new_vertex_cnt, new_rule_cnt = compress(
                vlist, elist, threshold, max_depth, min_edge, min_pair_frequency,
                self.compression_backend, compression_threads, compression_rounds, verbose)
            self.vertex_cnt = new_vertex_cnt
            self.rule_cnt = new_rule_cnt
            self.edge_cnt = new_elist.shape[0]
            src, dst = csr2coo(new_vlist, new_elist)
            if normalize:
                edge_weight = gcn_norm_coo_compress(src, dst, norm_degree, self.vertex_cnt, self.rule_cnt)
            else:
                edge_weight = np.ones(self.edge_cnt, dtype=np.float32)
            edge_mask, step = gen_mask_edge(src, dst, self.vertex_cnt, self.rule_cnt)
            if verbose:
                print("step:{}".format(step))
            self.step = step
            pairs = torch.from_numpy(np.vstack((src, dst)))
            weights = torch.from_numpy(edge_weight)
            self.edge_index, self.edge_weight = [], []
            for i in range(step):
                mask = torch.from_numpy(edge_mask[i])
                self.edge_index.append(torch.stack((pairs[0][mask], pairs[1][mask]), 0))
                self.edge_weight.append(weights[mask])
        else:
            raise ValueError('graph_type must be "coo" or "csr"')

    def __repr__(self):
        return 'CompressgnnData(vertex_cnt:"%s", rule_cnt:"%s", edge_cnt:"%s", step:"%s", graph_type:"%s")' % (
            self.vertex_cnt, self.rule_cnt, self.edge_cnt, self.step, self.graph_type)

    def to(self, device):
        self.x = self.x.to(device)
        self.y = self.y.to(device)
        self.train_mask = self.train_mask.to(device)
        self.vaild_mask = self.vaild_mask.to(device)
        self.test_mask = self.test_mask.to(device)
        if self.graph_type == "coo":
            for i in range(self.step):
                self.edge_index[i] = self.edge_index[i].to(device)
                self.edge_weight[i] = self.edge_weight[i].to(device)
        else:
            self.edge_index = self.edge_index.to(device)
        return self
