// CSR -> CSC on the device, in the order SparseTensor.csc() gives (reference
// layer/CompressgnnSPMM.py:68-70, loader/compress_graph.py:21-35 rely on it): entries
// sorted by column, ties in storage order, i.e. by row and then by position in the row.
//
// The entries are numbered in storage order and sorted by column with the library's own
// stable LSD radix sort (radix_sort.h; the payload of a key is its position), limited to the
// bits the column numbers occupy; the sorted position p then takes the row and value of
// entry perm[p], and colptr[c] is the first sorted position whose column is >= c.  Nothing
// here depends on timing: the result is the same array, bit for bit, as the host routine
// cgnn_csr_transpose produces.
#include "common.h"
#include "radix_sort.h"

namespace cgnn {
namespace {

constexpr int64_t kTransposeLimit = (int64_t)INT32_MAX - 65536;

struct TransposeWorkspace {
    size_t keys_in, keys_out, pos_out, tmp_keys, tmp_pos, counters, total;
};

TransposeWorkspace transpose_workspace(int64_t nnz) {
    TransposeWorkspace w{};
    const size_t arr = align_up((size_t)nnz * sizeof(int32_t), 256);
    w.keys_in = 0;
    w.keys_out = arr;
    w.pos_out = 2 * arr;
    w.tmp_keys = 3 * arr;
    w.tmp_pos = 4 * arr;
    w.counters = 5 * arr;
    w.total = 5 * arr + align_up(radix_sort_counter_bytes(nnz), 256);
    return w;
}

// keys[e] = column of entry e (the sort numbers the entries itself); flag is raised for a
// column outside [0, cols).
__global__ void transpose_keys_kernel(const int64_t *__restrict__ col, int64_t nnz, int64_t cols,
                                      int32_t *__restrict__ keys, int32_t *__restrict__ bad) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz;
         e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t c = col[e];
        if (c < 0 || c >= cols) {
            *bad = 1;  // every writer stores the same value
            keys[e] = 0;
        } else {
            keys[e] = (int32_t)c;
        }
    }
}

// Row and value (a 4- or 8-byte word W) of the entry that lands at sorted position p.
template <typename W>
__global__ void transpose_fill_kernel(const int64_t *__restrict__ rowptr, int64_t rows, int64_t nnz,
                                      const int32_t *__restrict__ perm, const W *__restrict__ val,
                                      int64_t *__restrict__ row_out, W *__restrict__ val_out) {
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < nnz;
         p += (int64_t)gridDim.x * blockDim.x) {
        const int64_t e = perm[p];
        int64_t lo = 0, hi = rows;  // invariant: rowptr[lo] <= e < rowptr[hi]
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if (rowptr[mid] <= e) lo = mid;
            else hi = mid;
        }
        row_out[p] = lo;
        if (val) val_out[p] = val[e];
    }
}

// colptr[c] = first sorted position whose column is >= c, for c = 0..cols.
__global__ void transpose_colptr_kernel(const int32_t *__restrict__ sorted_col, int64_t nnz, int64_t cols,
                                        int64_t *__restrict__ colptr) {
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c <= cols;
         c += (int64_t)gridDim.x * blockDim.x) {
        int64_t lo = 0, hi = nnz;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if ((int64_t)sorted_col[mid] < c) lo = mid + 1;
            else hi = mid;
        }
        colptr[c] = lo;
    }
}

__global__ void transpose_clear_flag_kernel(int32_t *flag) { *flag = 0; }

unsigned transpose_grid(int64_t n) {
    const int64_t b = ceil_div(n, kBlock);
    return (unsigned)(b > 65536 ? 65536 : (b < 1 ? 1 : b));
}

}  // namespace
}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_csr_transpose_workspace_bytes(int64_t nnz) {
    if (nnz <= 0 || nnz >= kTransposeLimit) return 0;
    return transpose_workspace(nnz).total;
}

extern "C" int cgnn_csr_transpose_device(int64_t rows, int64_t cols, int64_t nnz, const int64_t *rowptr,
                                         const int64_t *col, int dtype, const void *val, int64_t *colptr_out,
                                         int64_t *row_out, void *val_out, int32_t *bad_column,
                                         void *workspace, size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(dtype == CGNN_F32 || dtype == CGNN_F64, "cgnn_csr_transpose_device: dtype must be f32 or f64");
    CGNN_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "cgnn_csr_transpose_device: negative size");
    CGNN_REQUIRE(rows < kTransposeLimit && cols < kTransposeLimit && nnz < kTransposeLimit,
                 "cgnn_csr_transpose_device: rows/cols/nnz must be below 2^31 - 65536");
    CGNN_REQUIRE(colptr_out != nullptr && bad_column != nullptr, "cgnn_csr_transpose_device: null output");
    CGNN_REQUIRE(nnz == 0 || (rowptr && col && row_out), "cgnn_csr_transpose_device: null array");
    CGNN_REQUIRE(nnz == 0 || val == nullptr || val_out != nullptr, "cgnn_csr_transpose_device: values without output");
    hipLaunchKernelGGL(transpose_clear_flag_kernel, dim3(1), dim3(1), 0, stream, bad_column);
    if (nnz == 0) {
        hipLaunchKernelGGL(transpose_colptr_kernel, dim3(transpose_grid(cols + 1)), dim3(kBlock), 0, stream,
                           (const int32_t *)nullptr, (int64_t)0, cols, colptr_out);
        return check_launch("csr_transpose_device");
    }
    const TransposeWorkspace w = transpose_workspace(nnz);
    if (workspace == nullptr || workspace_bytes < w.total) {
        set_error("cgnn_csr_transpose_device: workspace of %zu bytes needed, %zu given", w.total, workspace_bytes);
        return CGNN_EWORKSPACE;
    }
    char *base = static_cast<char *>(workspace);
    auto at = [&](size_t off) { return reinterpret_cast<int32_t *>(base + off); };
    int32_t *keys_in = at(w.keys_in), *keys_out = at(w.keys_out), *pos_out = at(w.pos_out);
    hipLaunchKernelGGL(transpose_keys_kernel, dim3(transpose_grid(nnz)), dim3(kBlock), 0, stream, col, nnz, cols,
                       keys_in, bad_column);
    int bits = 1;
    while (bits < 31 && ((int64_t)1 << bits) < cols) ++bits;
    const int rc = radix_sort_positions(keys_in, nnz, bits, keys_out, pos_out, at(w.tmp_keys), at(w.tmp_pos),
                                        base + w.counters, stream);
    if (rc != CGNN_OK) return rc;
    if (dtype == CGNN_F64)
        hipLaunchKernelGGL(transpose_fill_kernel<uint64_t>, dim3(transpose_grid(nnz)), dim3(kBlock), 0, stream, rowptr,
                           rows, nnz, pos_out, static_cast<const uint64_t *>(val), row_out,
                           static_cast<uint64_t *>(val_out));
    else
        hipLaunchKernelGGL(transpose_fill_kernel<uint32_t>, dim3(transpose_grid(nnz)), dim3(kBlock), 0, stream, rowptr,
                           rows, nnz, pos_out, static_cast<const uint32_t *>(val), row_out,
                           static_cast<uint32_t *>(val_out));
    hipLaunchKernelGGL(transpose_colptr_kernel, dim3(transpose_grid(cols + 1)), dim3(kBlock), 0, stream, keys_out,
                       nnz, cols, colptr_out);
    return check_launch("csr_transpose_device");
}
