/*
 * compressgnn_abi.h -- C ABI of the MI355X (gfx950) device library libcgnn_hip.so.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream; none takes
 * a framework type, none allocates device memory and none synchronises with the host
 * unless its comment says so.  All launches go to the stream that is passed
 * (NULL = the device's null stream) on the device that is current in the calling
 * thread.  Return value: CGNN_OK (0) or a CGNN_E* code; cgnn_last_error() then holds
 * a message for the calling thread.
 *
 * The comments name the interface of the reference implementation
 * (ZhengChenCS/CompressGNN, paths relative to its root) that each entry replaces.
 *
 * Index arrays on the device are int32 (row counts and non-zero counts must be below
 * 2^31); offsets into feature matrices are computed in 64 bits.  Feature matrices are
 * dense row-major with row stride F.
 */
#ifndef COMPRESSGNN_ABI_H
#define COMPRESSGNN_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t *cgnn_stream_t; /* == hipStream_t */

enum cgnn_status {
    CGNN_OK = 0,
    CGNN_EINVAL = 1,       /* bad argument (shape, null pointer, range)          */
    CGNN_EWORKSPACE = 2,   /* workspace missing or smaller than *_workspace_bytes */
    CGNN_ELAUNCH = 3,      /* HIP reported an error at launch                     */
    CGNN_EUNSUPPORTED = 4  /* dtype / size outside what the kernels cover         */
};

enum cgnn_dtype { CGNN_F32 = 0, CGNN_F64 = 1 };

/* Which SpMM schedule to run.
 *   ROW: one lane group per row, entries of a row summed in ascending order
 *        (bit-identical to the sequential CPU sum of src/runtime/csrc/sparse/cpu/spmm_cpu.cpp:48-68).
 *   NNZ: fixed-length runs of non-zeros per lane group, rows that straddle runs are
 *        completed by an ordered fix-up pass (deterministic, no atomics).
 *   AUTO: chosen from cgnn_csr.max_row_nnz and the mean row length.
 * These replace the six CUDA methods of src/runtime/csrc/sparse/cuda/spmm_gpu.cu:27-99
 * and the Python heuristic layer/CompressgnnSPMM.py:14-19. */
enum cgnn_spmm_kernel { CGNN_SPMM_AUTO = 0, CGNN_SPMM_ROW = 1, CGNN_SPMM_NNZ = 2 };

/* A CSR block resident on the device.  rowidx[e] is the row of non-zero e
 * (non-decreasing); it is needed by the NNZ schedule only and may be NULL when the
 * ROW schedule is requested.  val == NULL means every stored value is 1. */
typedef struct cgnn_csr {
    int64_t rows;
    int64_t cols;
    int64_t nnz;
    const int32_t *rowptr; /* [rows+1] */
    const int32_t *colidx; /* [nnz]    */
    const int32_t *rowidx; /* [nnz] or NULL */
    const void *val;       /* [nnz] of the call's dtype, or NULL */
    int32_t max_row_nnz;   /* longest row, 0 if unknown (AUTO then picks NNZ) */
    int32_t seg_nnz;       /* NNZ schedule: non-zeros per lane group, 0 = default */
    /* Optional row permutation (NULL = none).  The arrays above then describe the rows in
     * a stored order chosen for locality (rows that gather the same columns next to each
     * other): stored row g is row rowmap[g] of Y.  Results are unchanged.  The workgroups
     * of such a block are numbered so that consecutive stored rows land on the same XCD
     * (the eight L2 caches of an MI355X are private). */
    const int32_t *rowmap; /* [rows] or NULL */
    /* NNZ schedule, optional (NULL = the fix-up pass looks at every run): the rows that the
     * runs cut and the rows without entries, ascending, as numbers of stored rows.  With run
     * length K = cgnn_spmm_run_length(A), row r is cut when rowptr[r+1] - rowptr[r] > K and
     * (rowptr[r] / K + 1) * K < rowptr[r+1] (integer division: the row is longer than a run and a
     * multiple of K lies strictly inside it; shorter rows are never cut).  Both lists
     * follow from rowptr and K alone and must be exact when given (they are not checked);
     * empty_rows may be NULL only if n_empty_rows is 0.  Results are unchanged. */
    const int32_t *cut_rows;   /* [n_cut_rows] */
    const int32_t *empty_rows; /* [n_empty_rows] */
    int32_t n_cut_rows, n_empty_rows;
    /* NNZ schedule, optional (NULL = every lane group finds its run from rowidx and rowptr, two
     * dependent loads before it can read its first entry): the first non-zero of every run,
     * [ceil(nnz / K) + 1] with K = cgnn_spmm_run_length(A).  run_start[s] for the position
     * e = s * K is nnz if e >= nnz, else rowptr[r] if row r = rowidx[e] has at most K entries (a short
     * row is never cut: the run begins with it), else e.  Must be exact when given (not checked).
     * Results are unchanged. */
    const int32_t *run_start;
} cgnn_csr;

const char *cgnn_last_error(void);
const char *cgnn_version(void);

/* ------------------------------------------------------------------ SpMM ---- */

/* The schedule CGNN_SPMM_AUTO stands for on a block of this shape that has rowidx (a block
 * without rowidx always takes the ROW schedule under AUTO): lets a caller build rowidx, which the
 * NNZ schedule alone reads, only for the blocks that will use it. */
int cgnn_spmm_schedule(int64_t rows, int64_t nnz, int32_t max_row_nnz, int kernel);

/* Non-zeros per run of the NNZ schedule for this block (seg_nnz, or the default, rounded up to
 * what the kernels take). */
int cgnn_spmm_run_length(const cgnn_csr *A);

/* Fills run_start[ceil(nnz / K) + 1] (K = cgnn_spmm_run_length(A)) for a block that has rowidx: the
 * optional table of cgnn_csr.run_start, as defined there.  No counterpart in the reference. */
int cgnn_spmm_run_starts(const cgnn_csr *A, int32_t *run_start, cgnn_stream_t stream);

/* Bytes of scratch cgnn_spmm needs for this block, feature width and schedule
 * (the carry-out rows of the NNZ schedule).  0 for the ROW schedule. */
size_t cgnn_spmm_workspace_bytes(const cgnn_csr *A, int64_t F, int dtype, int kernel);

/* Y[rows x F] (+)= A * X[cols x F].
 * accumulate == 0: every row of Y is written (empty rows become 0);
 * accumulate != 0: Y += A*X, rows without entries are left untouched, and Y may be
 * the same buffer as X provided no row that is written is also read (the in-place
 * rule-level update of layer/CompressgnnSPMM.py:56-58).
 * Replaces spmm_func / spmm_cuda: src/runtime/csrc/sparse/spmm.cpp:11-22,
 * src/runtime/csrc/sparse/cuda/spmm_gpu.cu:8-107. */
int cgnn_spmm(const cgnn_csr *A, int dtype, const void *X, void *Y, int64_t F,
              int accumulate, int kernel, void *workspace, size_t workspace_bytes,
              cgnn_stream_t stream);

/* cgnn_spmm with the scratch of the nnz schedule inside the library: no workspace argument, and
 * the call allocates nothing (no hipMalloc, no hipFree, no allocating library routine).  It has
 * no counterpart in the reference; it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation.  X, Y and the block are the
 * caller's as in cgnn_spmm, and the result is the same bit for bit.  The scratch is one array of
 * cgnn_spmm_static_scratch_bytes() bytes (64 MiB) in the library's device image; each GPU the
 * library runs on holds its copy until the process ends.  A product whose
 * cgnn_spmm_workspace_bytes exceeds that is refused with CGNN_EWORKSPACE (at F = 128 and the
 * default run length that is about 8 M non-zeros in the nnz schedule; the row schedule needs no
 * scratch and has no limit).  All calls on one GPU share the one array: calls that overlap
 * in time on the same GPU (two streams, two threads) race on it.
 * cgnn_spmm_static_init() looks up the array's address on the device that is current in the
 * calling thread (hipGetSymbolAddress, which may make the runtime load the library's device
 * image there: not an operation a stream capture can record).  cgnn_spmm_static does the same on
 * its first call on a device; a caller that captures, or that must not trigger the load inside
 * its loop, calls cgnn_spmm_static_init once per device beforehand.  After that a call launches
 * kernels and nothing else. */
size_t cgnn_spmm_static_scratch_bytes(void);
int cgnn_spmm_static_init(void);
int cgnn_spmm_static(const cgnn_csr *A, int dtype, const void *X, void *Y, int64_t F,
                     int accumulate, int kernel, cgnn_stream_t stream);

/* Two-source product in one pass: A has `cols` columns; a column c < split gathers
 * row c of X0, a column c >= split gathers row c - split of X1.  Every row of Y is
 * written as (0 + S1) + S0 with S1 / S0 the sums over the row's X1 / X0 entries, each
 * in storage order -- the value the two-call sequence
 *   out = spmm(v2r, rule_out, None); out = spmm(v2v, x, out)
 * of layer/CompressgnnSPMM.py:59-60 (84-85 in backward) produces when A's rows are
 * [v2v row | v2r row with columns shifted by split = vertex_cnt], without writing Y
 * twice or reading it back.  A->val must not be NULL.  Workspace as for cgnn_spmm. */
int cgnn_spmm_dual(const cgnn_csr *A, int64_t split, int dtype, const void *X0, const void *X1,
                   void *Y, int64_t F, int kernel, void *workspace, size_t workspace_bytes,
                   cgnn_stream_t stream);

/* Widen-free preparation of a CSR given as int64 tensors (the layout
 * src/runtime/csrc/sparse/cuda/spmm_gpu.cu:38-46 reads): converts rowptr/col to
 * int32 and writes the row of every non-zero.  Any of the outputs may be NULL. */
int cgnn_csr_prepare_i64(int64_t rows, int64_t nnz, const int64_t *rowptr64,
                         const int64_t *col64, int32_t *rowptr32, int32_t *col32,
                         int32_t *rowidx, cgnn_stream_t stream);

/* Column numbers of a block composed with a cluster assignment: out[e] = narrow_ids[colidx[e]]
 * where colidx[e] < first_cols, colidx[e] otherwise.  With these columns a product gathers row
 * ids[c] of a matrix of representatives where the block's own columns would gather row c of the
 * N x F matrix reps[ids] -- the rows Compressgnn_Reconstruct writes
 * (layer/CompressgnnReconstruct.py:34-42) and the next propagation reads
 * (layer/CompressgnnPropagation.py:62-67) -- so that matrix need not exist.  No counterpart in the
 * reference, whose layers hand each other dense tensors.  narrow_ids (first_cols entries, every
 * one in [0, groups) of the matrix of representatives) comes from cgnn_narrow_ids, which turns
 * the int64 ids of an assignment into int32, replaces an id outside [0, groups) by the nearest
 * valid one and stores 1 to *bad_id (may be NULL) when it meets one.  colidx and out: 16-byte
 * aligned. */
int cgnn_narrow_ids(int64_t n, const int64_t *ids, int64_t groups, int32_t *narrow_ids, int32_t *bad_id,
                    cgnn_stream_t stream);
int cgnn_csr_compose_columns(int64_t nnz, const int32_t *colidx, int64_t first_cols, const int32_t *narrow_ids,
                             int32_t *out, cgnn_stream_t stream);

/* rowidx[e] = row of non-zero e, from an int32 rowptr. */
int cgnn_csr_expand_rows(int64_t rows, int64_t nnz, const int32_t *rowptr,
                         int32_t *rowidx, cgnn_stream_t stream);

/* CSR -> CSC of a block given as int64 tensors on the device, in the order
 * SparseTensor.csc() gives (layer/CompressgnnSPMM.py:68-70 transposes every block of the
 * compressed graph that way for the backward pass; loader/compress_graph.py:21-35 relies on
 * the order): entries sorted by column, ties in storage order.  colptr_out has cols + 1
 * entries, row_out and val_out nnz; val (dtype CGNN_F32 or CGNN_F64) may be NULL.
 * *bad_column (device) is set to 1 if a column lies outside [0, cols) and to 0 otherwise;
 * the outputs are meaningless then.  Same arrays, bit for bit, as cgnn_csr_transpose of
 * the host library. */
size_t cgnn_csr_transpose_workspace_bytes(int64_t nnz);
int cgnn_csr_transpose_device(int64_t rows, int64_t cols, int64_t nnz, const int64_t *rowptr,
                              const int64_t *col, int dtype, const void *val, int64_t *colptr_out,
                              int64_t *row_out, void *val_out, int32_t *bad_column,
                              void *workspace, size_t workspace_bytes, cgnn_stream_t stream);

/* The batch pair merger on the device: what the reference's optional GPU compressor does
 * (src/offline/bindings/batch_cuda.cpp:3-9 -> compressgraph::compress_cuda, whose source is
 * not part of the reference tree; loader/compression_backend.py:24-40 calls it).  vlist
 * (V + 1 entries) and elist (E entries, columns in [0, V)) are int64 arrays on the device.
 * Result, the same arrays as cgnn_compress_csr_batch of the host library gives: out_ptr
 * (capacity V + E/2 + 2) holds the V + R + 1 row starts, out_col (capacity E) the vertex
 * rows written with vertex and rule ids, followed by the two children of every rule;
 * host_summary[0] = R, host_summary[1] = entries of out_col.  Offline work: the call waits
 * for the device (three small reads per round) and returns when the arrays are complete. */
size_t cgnn_compress_batch_workspace_bytes(int64_t V, int64_t E);
int cgnn_compress_csr_batch_device(int64_t V, int64_t E, const int64_t *vlist, const int64_t *elist,
                                   int rounds, int min_pair_frequency, int32_t *out_ptr,
                                   int32_t *out_col, int64_t *host_summary, void *workspace,
                                   size_t workspace_bytes, cgnn_stream_t stream);

/* ------------------------------------------------- transformation compression -- */

/* Scratch for cgnn_lsh_scan: bytes needed for 2^bits buckets. */
size_t cgnn_lsh_scan_workspace_bytes(int bits);

/* Step 1 of the assignment (src/runtime/csrc/cluster/cuda/cluster_kernel.cu:136-142,
 * CPU twin src/runtime/csrc/cluster/cpu/cluster_cpu.cpp:41-56): for every row i of
 * X[N x F], h_j = sum_k X[i,k]*W[k,j] accumulated with fused multiply-add in
 * ascending k starting from 0, code = sum_j (h_j > 0) << (bits-1-j);
 * raw_code[i] = code and bucket_count[code] += 1.  bucket_count (2^bits int32) is
 * cleared by this call.  W is [F x bits] row-major. */
int cgnn_lsh_hash(int64_t N, int64_t F, int bits, int dtype, const void *X, const void *W,
                  int32_t *raw_code, int32_t *bucket_count, cgnn_stream_t stream);

/* bucket_count may be NULL: then only raw_code is produced (cgnn_lsh_group derives the
 * counts from the codes without any atomic update). */

/* Step 2: prefix[b] = number of occupied buckets with index <= b (inclusive scan,
 * cluster_kernel.cu:143-145).  prefix[2^bits - 1] is the number of active buckets;
 * the caller reads it back (the one host synchronisation of cluster_kernel.cu:147). */
int cgnn_lsh_scan(int bits, const int32_t *bucket_count, int32_t *prefix, void *workspace,
                  size_t workspace_bytes, cgnn_stream_t stream);

/* Step 3 (cluster_kernel.cu:51-59,149-150): ids[i] = prefix[raw_code[i]] (1-based,
 * int64) and counts[prefix[b]] = bucket_count[b] for occupied b.  counts has
 * active+1 entries and must be zero on entry (entry 0 stays 0). */
int cgnn_lsh_finish(int64_t N, int bits, const int32_t *raw_code, const int32_t *bucket_count,
                    const int32_t *prefix, int64_t *ids, int32_t *counts, cgnn_stream_t stream);

/* The bad_id argument of the entries that read caller-supplied cluster ids
 * (cgnn_cluster_members, cgnn_cluster_mean_backward, cgnn_reconstruct, cgnn_reconstruct_signs): a device int32, or
 * NULL.  The reference traps in the kernel on an id outside [0, groups)
 * (CUDA_KERNEL_ASSERT, cluster_kernel.cu:74,92); here such an id is treated as the nearest
 * valid one, so that no access leaves the arrays, and 1 is stored to *bad_id.  0 is never
 * stored: the caller clears the flag before a call, or a sequence of calls, and reads it
 * afterwards; the results of a flagged call are meaningless. */

/* Member lists of the clusters: a stable counting sort of the rows by id.
 * offsets[g] = first position of group g in perm (offsets has groups+1 entries),
 * perm[p] = row, sorted_id[p] = its id; rows of one group appear in ascending order.
 * This is the CSR the segmented reductions below run on; it replaces the per-element
 * float atomics of sum_features / reconstruct_grad (cluster_kernel.cu:60-69,98-108). */
size_t cgnn_cluster_members_workspace_bytes(int64_t N, int64_t groups);
int cgnn_cluster_members(int64_t N, int64_t groups, const int64_t *ids, int32_t *offsets,
                         int32_t *perm, int32_t *sorted_id, int32_t *bad_id, void *workspace,
                         size_t workspace_bytes, cgnn_stream_t stream);

/* Steps 2 and 3 and the member lists in one, from the raw codes alone (no bucket
 * counters): rows are sorted by code (stable), a run of equal codes is a group, and the
 * 1-based id of a group is the rank of its code.  Produces what cgnn_lsh_scan +
 * cgnn_lsh_finish + cgnn_cluster_members produce -- ids[N], counts[active+1] (entry 0 = 0),
 * offsets[active+2], perm[N], sorted_id[N] -- and summary[2] (device): summary[0] = active,
 * the number of groups, summary[1] = the size of the largest group.  counts needs room for min(N, 2^bits)+1 entries and offsets for one more; entries
 * beyond active+1 (active+2) are left untouched.  Replaces cluster_kernel.cu:143-150 and
 * the atomics of hash_ids (cluster_kernel.cu:41-59). */
size_t cgnn_lsh_group_workspace_bytes(int64_t N, int bits);
int cgnn_lsh_group(int64_t N, int bits, const int32_t *raw_code, int64_t *ids, int32_t *offsets,
                   int32_t *perm, int32_t *sorted_id, int32_t *counts, int32_t *summary,
                   void *workspace, size_t workspace_bytes, cgnn_stream_t stream);

/* reps[g,:] = (sum over members i of group g, ascending i, of X[i,:]) / max(counts[g],1).
 * max_members: size of the largest group if the caller knows it (it decides whether the
 * sums of very large groups need the multi-level carry reduction), 0 if not.  The
 * workspace size covers either case.
 * Replaces cluster_mean_cuda (cluster_kernel.cu:158-170). */
size_t cgnn_cluster_mean_workspace_bytes(int64_t N, int64_t F, int64_t groups, int dtype);
int cgnn_cluster_mean(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype, const void *X,
                      const int32_t *offsets, const int32_t *perm, const int32_t *sorted_id,
                      const int32_t *counts, void *reps, void *workspace,
                      size_t workspace_bytes, cgnn_stream_t stream);

/* dx[i,:] = grad[ids[i],:] / max(counts[ids[i]],1).  perm (the member list of
 * cgnn_cluster_members for these ids, or NULL) only sets the order in which rows are
 * produced: grouped by cluster, every row of grad is fetched from memory once.
 * Replaces cluster_mean_backward_cuda (cluster_kernel.cu:171-181). */
int cgnn_cluster_mean_backward(int64_t N, int64_t F, int64_t groups, int dtype, const void *grad,
                               const int64_t *ids, const int32_t *counts, const int32_t *perm,
                               void *dx, int32_t *bad_id, cgnn_stream_t stream);

/* out[i,:] = act(reps[ids[i],:] + bias), act(v) = (relu && v < 0) ? 0 : v; bias may be
 * NULL; perm as above (NULL = rows in natural order).
 * Replaces cluster_reconstruct_cuda (cluster_kernel.cu:182-195). */
int cgnn_reconstruct(int64_t N, int64_t F, int64_t groups, int dtype, const void *reps,
                     const int64_t *ids, const int32_t *perm, const void *bias, int relu,
                     void *out, int32_t *bad_id, cgnn_stream_t stream);

/* reps_grad[g,:] = sum over members i of g (ascending) of
 * ((relu && output[i,:] <= 0) ? 0 : grad[i,:]).  max_members as for cgnn_cluster_mean.
 * Replaces cluster_reconstruct_backward_cuda (cluster_kernel.cu:196-208). */
int cgnn_reconstruct_backward(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype, const void *grad,
                              const void *output, const int32_t *offsets, const int32_t *perm,
                              const int32_t *sorted_id, int relu, void *reps_grad,
                              void *workspace, size_t workspace_bytes, cgnn_stream_t stream);

/* The ReLU mask as one bit per element.  cgnn_reconstruct_signs is cgnn_reconstruct with relu = 1
 * that also writes signs[i * W + f / 32], W = cgnn_sign_words(F) = ceil(F / 32): bit f % 32 is set
 * unless out[i,f] <= 0 (bits past F are clear).  cgnn_reconstruct_backward_signs is
 * cgnn_reconstruct_backward with relu = 1 that drops grad[i,f] where the bit is clear, so it reads
 * N * W words in place of the N x F saved output and gives the same reps_grad bit for bit.
 * No counterpart in the reference, whose layer keeps the whole output for its backward pass
 * (layer/CompressgnnReconstruct.py:16-26, cluster_kernel.cu:196-208). */
int64_t cgnn_sign_words(int64_t F);
int cgnn_reconstruct_signs(int64_t N, int64_t F, int64_t groups, int dtype, const void *reps,
                           const int64_t *ids, const int32_t *perm, const void *bias, void *out,
                           uint32_t *signs, int32_t *bad_id, cgnn_stream_t stream);
int cgnn_reconstruct_backward_signs(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype,
                                    const void *grad, const uint32_t *signs, const int32_t *offsets,
                                    const int32_t *perm, const int32_t *sorted_id, void *reps_grad,
                                    void *workspace, size_t workspace_bytes, cgnn_stream_t stream);

/* ---------------------------------------- neighbour sampling on a compressed graph -- */

/* The work of the reference's CPU module compressgnn_sample
 * (src/sample/csrc/function.cpp:7-9: neighbor_sample_cg_sim = neighbor_sample_sim_impl,
 * src/sample/csrc/neighbor_sample.h:27-131, over get_neighbor / get_neighbor_list of
 * src/sample/csrc/storage_api.h:6-118; neighbor_sample_ori_impl, :134-211, is the graph without
 * rules) as device entry points.  One layer: cgnn_sample_count -> cgnn_exclusive_sum_i32 ->
 * (the caller reads the total and sizes the outputs) -> cgnn_sample_fill -> cgnn_sample_relabel;
 * cgnn_sample_relabel_begin once per call before the first layer. */
#define CGNN_SAMPLE_MAX_LEVELS 16

/* The blocks of a CompressGraph as the sampler reads them: int64 arrays on the device, the
 * tensors of loader/compress_graph.py:21-43 (csr() of v2v_graph, v2r_graph, r2v_graph and of
 * every r2r level, vertex_degree, rule_degree).  A graph without rules (rule_cnt = 0, levels = 0)
 * may leave everything but v2v_ptr / v2v_idx NULL: v2v is then (colptr, row) and the degree of
 * a vertex is the length of its row. */
typedef struct cgnn_sample_graph {
    int64_t vertex_cnt, rule_cnt;
    int32_t levels;                       /* r2r levels, at most CGNN_SAMPLE_MAX_LEVELS */
    const int64_t *v2v_ptr, *v2v_idx;     /* [vertex_cnt + 1], [nnz] */
    const int64_t *v2r_ptr, *v2r_idx;     /* [vertex_cnt + 1], [nnz]: rules in [0, rule_cnt) */
    const int64_t *r2v_ptr, *r2v_idx;     /* [rule_cnt + 1], [nnz] */
    const int64_t *r2r_ptr[CGNN_SAMPLE_MAX_LEVELS]; /* [rule_cnt + 1] per level */
    const int64_t *r2r_idx[CGNN_SAMPLE_MAX_LEVELS];
    const int64_t *v_degree, *r_degree;   /* expanded degrees (gen_degree.h:10-85) */
} cgnn_sample_graph;

/* *status (device int32; cleared by cgnn_sample_relabel_begin) after the kernels of a call: */
enum cgnn_sample_status {
    CGNN_SAMPLE_OK = 0,
    CGNN_SAMPLE_OUT_OF_RANGE = 1, /* a random position beyond what the descent through the rules finds:
                                     where the reference throws std::out_of_range (storage_api.h:69) */
    CGNN_SAMPLE_BAD_VERTEX = 2,   /* a vertex id outside [0, vertex_cnt) in the input or in the graph */
    CGNN_SAMPLE_TOO_MANY = 3      /* more than 2^31 - 2 neighbours in one layer */
};

/* out[0] = 0, out[i + 1] = in[0] + ... + in[i]: n + 1 entries.  A sum beyond 2^31 - 2 is
 * stored as INT32_MAX and reported through *status (may be NULL). */
size_t cgnn_exclusive_sum_workspace_bytes(int64_t n);
int cgnn_exclusive_sum_i32(int64_t n, const int32_t *in, int32_t *out, int32_t *status, void *workspace,
                           size_t workspace_bytes, cgnn_stream_t stream);

/* counts[i] = number of neighbours that frontier vertex i contributes to the layer: 0 for a
 * vertex of degree 0, the length of its full neighbour list when fanout >= its degree, else
 * fanout (neighbor_sample.h:88-99). */
int cgnn_sample_count(const cgnn_sample_graph *graph, int64_t n, const int64_t *frontier, int64_t fanout,
                      int32_t *counts, int32_t *status, cgnn_stream_t stream);

/* Writes the neighbours of frontier vertex i to neighbors[offsets[i] .. offsets[i + 1]) and
 * first_position + i (its position among the samples) to the same range of sources.  A full
 * list comes in the order of get_neighbor_list (storage_api.h:72-118); a sampled one holds the
 * neighbours at the positions the selection loop of neighbor_sample.h:112-118 picks, in the
 * order it picks them, each resolved as get_neighbor does (storage_api.h:6-70).  The loop's
 * draws come from a counter-based generator keyed by (seed, layer, first_position + i, step).
 * picks: scratch of offsets[n] entries. */
int cgnn_sample_fill(const cgnn_sample_graph *graph, int64_t n, const int64_t *frontier, int64_t fanout,
                     const int32_t *offsets, int64_t first_position, int64_t layer, uint64_t seed,
                     int64_t *neighbors, int64_t *sources, int64_t *picks, int32_t *status,
                     cgnn_stream_t stream);

/* Start of a sampling call: clears *status, marks every vertex as not yet numbered
 * (local_of and seen_at: int32[vertex_cnt] each) and numbers the input vertices 0, 1, ... (of
 * equal ones the first counts, as the hash map of neighbor_sample.h:72-76 has it). */
int cgnn_sample_relabel_begin(int64_t vertex_cnt, int64_t n_input, const int64_t *input, int32_t *local_of,
                              int32_t *seen_at, int32_t *status, cgnn_stream_t stream);

/* Local numbers for the `total` neighbours of a layer (neighbor_sample.h:100-106,119-125): a
 * vertex numbered before keeps its number; the others take base, base + 1, ... in the order
 * of their first occurrence and are appended to samples at those positions (samples needs room
 * for base + total entries).  numbers[t] = local number of neighbors[t]; *new_count (device) =
 * vertices added. */
size_t cgnn_sample_relabel_workspace_bytes(int64_t total);
int cgnn_sample_relabel(int64_t total, const int64_t *neighbors, int64_t base, int32_t *local_of,
                        int32_t *seen_at, int64_t *samples, int64_t *numbers, int64_t *new_count,
                        void *workspace, size_t workspace_bytes, cgnn_stream_t stream);

/* --------------------------------------------------------------- utilities ---- */

/* A plain device-to-device copy kernel of n bytes (n % 16 == 0); the calibration
 * kernel for scaling profiler byte counters. */
int cgnn_copy_bytes(const void *src, void *dst, size_t n, cgnn_stream_t stream);

/* A plain streaming read of n bytes (n % 16 == 0) that stores nothing (sink: 4 bytes of
 * device memory, practically never written): the read rate the memory system sustains,
 * which is what the gather-bound kernels are compared with. */
int cgnn_read_bytes(const void *src, size_t n, void *sink, cgnn_stream_t stream);

/* A plain streaming write of n bytes of zeros (n % 16 == 0): the write rate the memory
 * system sustains, which is what the write-bound kernels (reconstruct, the gradient of the
 * means) are compared with. */
int cgnn_fill_bytes(void *dst, size_t n, cgnn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* COMPRESSGNN_ABI_H */
