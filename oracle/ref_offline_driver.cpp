// Build-side driver for oracle/_ref: registers the reference's header-only offline
// routines (included from the reference checkout, not copied) under the module name
// compressgnn_offline_ref so that tests/golden/make_golden.py can record their outputs.
// The reference's own module definition (src/offline/csrc/function.cpp) cannot be
// linked because it requires the un-vendored CompressGraph compressor; that
// compressor is left out here, nothing stands in for it.
#include "add_self_loop.h"
#include "convert.h"
#include "depth_filter.h"
#include "filter.h"
#include "gen_degree.h"
#include "norm.h"
#include "partition.h"
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

PYBIND11_MODULE(compressgnn_offline_ref, m) {
    m.def("gen_vertex_order_csr", &gen_vertex_order_csr);
    m.def("gen_vertex_order_csc", &gen_vertex_order_csc);
    m.def("filter_csr", &filter_csr);
    m.def("depth_filter_csr", &depth_filter_csr);
    m.def("coo2csr", &coo2csr);
    m.def("csr2coo", &csr2coo);
    m.def("add_self_loop_csr", &add_self_loop_csr);
    m.def("get_norm_degree", &get_norm_degree);
    m.def("gcn_norm_csr", &gcn_norm_csr);
    m.def("gcn_norm_csr_compress", &gcn_norm_csr_compress);
    m.def("hybird_partition", &hybird_partition);
    m.def("topo_partition", &topo_partition);
    m.def("gen_degree", &gen_degree);
    m.def("add_self_loop_coo", &add_self_loop_coo);
    m.def("gcn_norm_coo_compress", &gcn_norm_coo_compress);
    m.def("gen_edge_order", &gen_edge_order);
    m.def("gen_mask_edge", &gen_mask_edge);
}
