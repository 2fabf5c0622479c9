/*
 * compressgnn_prep.h -- C ABI of the host-side graph preparation library
 * libcgnn_prep.so (plain C++, no GPU code): everything that builds the CompressGraph
 * blocks the device kernels consume.  All pointers are host pointers; index arrays are
 * int64, weights float32, exactly the array types of the reference's offline module
 * (ZhengChenCS/CompressGNN src/offline/csrc/util.h:14 `VertexT int64_t`).
 *
 * Functions with outputs whose size is not known in advance return a cgnn_arrays
 * bundle (an ordered list of typed arrays owned by the library) that the caller reads
 * and then frees.  Functions return NULL / non-zero on error; cgnn_prep_last_error()
 * has the message.
 */
#ifndef COMPRESSGNN_PREP_H
#define COMPRESSGNN_PREP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cgnn_arrays cgnn_arrays;
enum cgnn_array_type { CGNN_ARR_I64 = 0, CGNN_ARR_F32 = 1, CGNN_ARR_I32 = 2 };

int cgnn_arrays_count(const cgnn_arrays *a);
int cgnn_arrays_type(const cgnn_arrays *a, int i);
int64_t cgnn_arrays_size(const cgnn_arrays *a, int i); /* elements */
const void *cgnn_arrays_data(const cgnn_arrays *a, int i);
int64_t cgnn_arrays_scalar(const cgnn_arrays *a, int i); /* i-th extra scalar result */
void cgnn_arrays_free(cgnn_arrays *a);
const char *cgnn_prep_last_error(void);

/* add_self_loop_csr (src/offline/csrc/add_self_loop.h:17-43): rows sorted ascending;
 * vertex v is inserted at its sorted place unless present.  -> [vlist, elist] */
cgnn_arrays *cgnn_add_self_loop_csr(int64_t V, const int64_t *vlist, const int64_t *elist);

/* get_norm_degree (src/offline/csrc/norm.h:20-45): out[v] = 1/sqrt(1e-6 + indegree(v)),
 * accumulated and rounded in float32. */
int cgnn_get_norm_degree(int64_t E, const int64_t *dst, int64_t V, float *out);

/* gcn_norm_csr_compress (norm.h:179-216): weight of edge (row -> dst) of the compressed
 * CSR: vertex->vertex d[row]*d[dst], vertex->rule d[row], rule->vertex d[dst], rule->rule 1. */
int cgnn_gcn_norm_csr_compress(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist,
                               const float *norm_degree, float *weight);

/* add_self_loop_coo (src/offline/csrc/add_self_loop.h:55-107): edges grouped by ascending
 * source, targets ascending within a source; (v, v) is inserted behind v's targets below
 * v unless present.  -> [src, dst] */
cgnn_arrays *cgnn_add_self_loop_coo(int64_t E, const int64_t *src, const int64_t *dst, int64_t V);

/* gcn_norm_coo_compress (norm.h:129-166): the edge weights of gcn_norm_csr_compress for
 * an edge list (src -> dst) over V vertices followed by R rules. */
int cgnn_gcn_norm_coo_compress(int64_t E, const int64_t *src, const int64_t *dst,
                               const float *norm_degree, int64_t V, int64_t R, float *weight);

/* gen_edge_order (src/offline/csrc/gen_mask.h:10-84), from which gen_mask_edge
 * (gen_mask.h:86-108) forms its phase masks: phase 0 = edges that leave a vertex, phase
 * k >= 1 = edges that leave a rule all of whose rule inputs arrived in phases < k.
 * -> [order (int32, E)]; scalar: number of phases. */
cgnn_arrays *cgnn_gen_edge_order(int64_t E, const int64_t *src, const int64_t *dst, int64_t V, int64_t R);

/* CSR -> CSC of a rows x cols matrix: entries ordered by column, then by row, ties in
 * original order (the order torch_sparse's SparseTensor.csc() yields, which
 * loader/CompressgnnData.py:180 and layer/CompressgnnSPMM.py:68-70 rely on).
 * value may be NULL.  -> [colptr (cols+1), row, value] */
cgnn_arrays *cgnn_csr_transpose(int64_t rows, int64_t cols, const int64_t *vlist,
                                const int64_t *elist, const float *value);

/* hybird_partition (src/offline/csrc/partition.h:14-110): splits the (V+R)-row matrix
 * whose rows list vertex columns first, then rule columns, into the four blocks.
 * -> [v2v_vlist, v2v_elist, v2v_value, v2r_*, r2v_*, r2r_*] (12 arrays) */
cgnn_arrays *cgnn_hybird_partition(int64_t total, const int64_t *vlist, const int64_t *elist,
                                   const float *value, int64_t V);

/* topo_partition (partition.h:112-216): level matrices of the rule->rule block, each
 * with R+1 row pointers.  -> 3 arrays per level; scalar 0 = number of levels. */
cgnn_arrays *cgnn_topo_partition(int64_t R, const int64_t *vlist, const int64_t *elist,
                                 const float *value);

/* gen_degree (src/offline/csrc/gen_degree.h:10-85).  level_vlists/level_elists are
 * arrays of `levels` pointers.  -> [vertex_degree (V), rule_degree (R)] */
cgnn_arrays *cgnn_gen_degree(int64_t V, int64_t R, const int64_t *v2v_vlist, const int64_t *v2r_vlist,
                             const int64_t *v2r_elist, const int64_t *r2v_vlist, int levels,
                             const int64_t *const *level_vlists,
                             const int64_t *const *level_elists);

/* filter_csr (src/offline/csrc/filter.h:80-118): inlines rules whose saving
 * (freq-1)(len-1)-1 is at most `threshold`.  -> [vlist, elist]; scalars: V, R'. */
cgnn_arrays *cgnn_filter_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist,
                             int threshold);

/* depth_filter_csr (src/offline/csrc/depth_filter.h:40-116).  -> [vlist, elist]; scalars V, R'. */
cgnn_arrays *cgnn_depth_filter_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist,
                                   int max_depth, int min_edge);

/* gen_vertex_order_csr (src/offline/csrc/gen_mask.h:180-233). -> [order (int32, V+R)]; scalar: depth. */
cgnn_arrays *cgnn_gen_vertex_order_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist);

/* gen_vertex_order_csc (gen_mask.h:111-174), the phase count CompressgnnData.step reports
 * (loader/CompressgnnData.py:177-179). -> [order (int32, V+R)]; scalar: phases. */
cgnn_arrays *cgnn_gen_vertex_order_csc(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist);

/* Batch pair-merging compressor: stands where the reference calls
 * compress_csr_batch(vlist, elist, threads, rounds, min_pair_frequency)
 * (loader/compression_backend.py:24-40; its implementation is a submodule that the
 * reference tree does not contain).  Contract kept: int32 outputs, vertex rows expand
 * (in order) to the input rows, every rule's children have smaller ids than the rule,
 * min_pair_frequency >= 3.  -> [vlist (int32), elist (int32)]; scalars: V, R. */
cgnn_arrays *cgnn_compress_csr_batch(int64_t V, const int64_t *vlist, const int64_t *elist,
                                     int threads, int rounds, int min_pair_frequency);

/* [A0 | A1]: row r of the result is row r of A0 followed by row r of A1 with its
 * columns shifted by col_offset (the vertex stage of the propagation reads the
 * vertex->vertex and vertex->rule blocks this way in one pass). -> [vlist, elist, value] */
cgnn_arrays *cgnn_csr_hstack(int64_t rows, const int64_t *vlist0, const int64_t *elist0, const float *value0,
                             const int64_t *vlist1, const int64_t *elist1, const float *value1,
                             int64_t col_offset);

/* A row order for locality: rows that share many columns follow each other (a depth-first
 * walk of the forest that ties every row to the row it shares most columns with; trees and
 * unrelated rows in the lexicographic order of their column lists).  The order depends on
 * the matrix only, not on the number of threads.  -> [order (int32, rows)]: position g of
 * the order holds row order[g]. */
cgnn_arrays *cgnn_csr_locality_order(int64_t rows, const int64_t *vlist, const int64_t *elist);

/* A block B (R rows) with the rule levels folded in: the result of the in-place updates
 * B[r] += sum_c L_k[r, c] * B[c], k = 0 .. levels-1 (layer/CompressgnnSPMM.py:56-58 applies
 * them as one product per level), as one matrix with the entries of a row merged by column.
 * Every level matrix is R x R and reads only rows it does not write.  -> [vlist, elist, value] */
cgnn_arrays *cgnn_csr_fold_levels(int64_t R, const int64_t *vlist, const int64_t *elist, const float *value,
                                  int levels, const int64_t *const *level_vlists,
                                  const int64_t *const *level_elists, const float *const *level_values);

/* The CSR with its rows rearranged: row g of the result is row order[g] of the input
 * (value may be NULL).  -> [vlist, elist, value] */
cgnn_arrays *cgnn_csr_permute_rows(int64_t rows, const int64_t *vlist, const int64_t *elist,
                                   const float *value, const int32_t *order);

/* Longest row, and a histogram of row lengths in powers of two:
 * hist[k] = rows with length in [2^(k-1), 2^k) for k >= 1, hist[0] = empty rows. */
int cgnn_csr_row_stats(int64_t rows, const int64_t *vlist, int64_t *max_row, int64_t hist[40]);

/* Seeded synthetic graphs (rows sorted, no duplicates, no self loops). -> [vlist, elist]
 * chung_lu: expected degrees follow a power law with the given exponent, scaled so the
 *           expected number of directed edges is target_edges.
 * copy_model: vertex t > 0 picks a prototype p < t uniformly, keeps each out-neighbour
 *           of p with probability copy_prob and adds uniformly random out-links so that
 *           the expected out-degree is avg_degree. */
cgnn_arrays *cgnn_gen_chung_lu(int64_t V, int64_t target_edges, double exponent, uint64_t seed);
cgnn_arrays *cgnn_gen_copy_model(int64_t V, double avg_degree, double copy_prob, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif /* COMPRESSGNN_PREP_H */
