// Member lists of the clusters: rows sorted by cluster id, ties in ascending row
// order.  The sort itself is rocPRIM's stable LSD radix sort (through hipCUB) on
// (id, row) pairs, limited to the bits the ids occupy; it runs once per assignment
// refresh, not per training step.  Everything else here is hand-written.
//
// cgnn_lsh_group derives ids, counts and member lists from the raw hash codes with the
// same sort: the dense id of a row is the rank of its code among the codes that occur, so
// sorting by code is sorting by id, the groups are the runs of equal codes and no counter
// is ever updated atomically (rows of a graph pile up in a few codes).
#include <hipcub/hipcub.hpp>

#include <algorithm>

#include "common.h"

namespace cgnn {
namespace {

// An id outside [0, groups) is filed under the nearest group that exists (the lists then
// index nothing beyond their arrays) and reported through the flag.
__global__ void members_keys_kernel(const int64_t *__restrict__ ids, int32_t *__restrict__ keys,
                                    int32_t *__restrict__ rows, int64_t N, int64_t groups,
                                    int32_t *__restrict__ bad_id) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
         i += (int64_t)gridDim.x * blockDim.x) {
        int64_t id = ids[i];
        if (id < 0 || id >= groups) {
            id = id < 0 ? 0 : groups - 1;
            if (bad_id) *bad_id = 1;  // every writer stores the same value
        }
        keys[i] = (int32_t)id;
        rows[i] = (int32_t)i;
    }
}

// offsets[g] = first position p with sorted_id[p] >= g (g = 0..groups).
__global__ void members_offsets_kernel(const int32_t *__restrict__ sorted_id, int64_t N,
                                       int32_t *__restrict__ offsets, int64_t groups) {
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g <= groups;
         g += (int64_t)gridDim.x * blockDim.x) {
        int64_t lo = 0, hi = N;
        while (lo < hi) {
            int64_t mid = (lo + hi) >> 1;
            if (sorted_id[mid] < g) lo = mid + 1;
            else hi = mid;
        }
        offsets[g] = (int32_t)lo;
    }
}

__global__ void iota_kernel(int32_t *__restrict__ rows, int64_t N) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
         i += (int64_t)gridDim.x * blockDim.x)
        rows[i] = (int32_t)i;
}

// head[p] = 1 where a run of equal codes starts.
__global__ void group_heads_kernel(const int32_t *__restrict__ sorted_code, int64_t N,
                                   int32_t *__restrict__ head, int32_t *__restrict__ summary) {
    if (blockIdx.x == 0 && threadIdx.x == 0) summary[1] = 0;  // running maximum of the group sizes
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < N;
         p += (int64_t)gridDim.x * blockDim.x)
        head[p] = (p == 0 || sorted_code[p] != sorted_code[p - 1]) ? 1 : 0;
}

// rank[p] (the inclusive count of heads) is the 1-based id of the row at sorted position p.
__global__ void group_finish_kernel(int64_t N, const int32_t *__restrict__ rank,
                                    const int32_t *__restrict__ head, const int32_t *__restrict__ perm,
                                    int64_t *__restrict__ ids, int32_t *__restrict__ offsets,
                                    int32_t *__restrict__ active) {
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < N;
         p += (int64_t)gridDim.x * blockDim.x) {
        const int32_t id = rank[p];
        ids[perm[p]] = id;
        if (head[p]) offsets[id] = (int32_t)p;
        if (p == 0) offsets[0] = 0;
        if (p == N - 1) {
            offsets[id + 1] = (int32_t)N;
            *active = id;
        }
    }
}

// summary[0] = number of groups (set by group_finish_kernel), summary[1] = largest group.
__global__ void group_counts_kernel(const int32_t *__restrict__ offsets, int32_t *__restrict__ summary,
                                    int32_t *__restrict__ counts, int64_t capacity) {
    const int64_t groups = min((int64_t)summary[0], capacity) + 1;
    int largest = 0;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups;
         g += (int64_t)gridDim.x * blockDim.x) {
        const int c = g == 0 ? 0 : offsets[g + 1] - offsets[g];
        counts[g] = c;
        largest = max(largest, c);
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) largest = max(largest, __shfl_xor(largest, d, kWave));
    if (threadIdx.x % kWave == 0 && largest > 0) atomicMax(summary + 1, largest);
}

__global__ void group_empty_kernel(int32_t *offsets, int32_t *counts, int32_t *summary) {
    offsets[0] = offsets[1] = 0;
    counts[0] = 0;
    summary[0] = summary[1] = 0;
}

int key_bits(int64_t groups) {
    int b = 1;
    while (((int64_t)1 << b) < groups) ++b;
    return b;
}

size_t sort_temp_bytes(int64_t N, int64_t groups) {
    size_t bytes = 0;
    hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, (const int32_t *)nullptr, (int32_t *)nullptr,
                                       (const int32_t *)nullptr, (int32_t *)nullptr, (int)N, 0,
                                       key_bits(groups), (hipStream_t) nullptr);
    return bytes;
}

size_t code_sort_temp_bytes(int64_t N, int bits) {
    size_t bytes = 0;
    hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, (const int32_t *)nullptr, (int32_t *)nullptr,
                                       (const int32_t *)nullptr, (int32_t *)nullptr, (int)N, 0,
                                       bits < 1 ? 1 : bits, (hipStream_t) nullptr);
    return bytes;
}

}  // namespace

size_t occupancy_scan_bytes(int64_t n);
int occupancy_scan(const int32_t *in, int64_t n, int32_t *out, void *scratch, hipStream_t stream);

}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_lsh_group_workspace_bytes(int64_t N, int bits) {
    if (N <= 0 || N >= INT32_MAX || bits < 0 || bits > 30) return 0;
    const size_t col = align_up((size_t)N * sizeof(int32_t), 256);
    // row numbers, sorted codes, run heads, scan scratch, sort scratch
    return 3 * col + occupancy_scan_bytes(N) + align_up(code_sort_temp_bytes(N, bits), 256);
}

extern "C" int cgnn_lsh_group(int64_t N, int bits, const int32_t *raw_code, int64_t *ids, int32_t *offsets,
                              int32_t *perm, int32_t *sorted_id, int32_t *counts, int32_t *summary,
                              void *workspace, size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && N < INT32_MAX, "cgnn_lsh_group: row count must be in [0, 2^31)");
    CGNN_REQUIRE(bits >= 0 && bits <= 30, "cgnn_lsh_group: bits must be in [0, 30]");
    CGNN_REQUIRE(offsets && counts && summary, "cgnn_lsh_group: null output");
    if (N == 0) {
        hipLaunchKernelGGL(group_empty_kernel, dim3(1), dim3(1), 0, stream, offsets, counts, summary);
        return check_launch("lsh_group");
    }
    CGNN_REQUIRE(raw_code && ids && perm && sorted_id, "cgnn_lsh_group: null array");
    if (workspace == nullptr || workspace_bytes < cgnn_lsh_group_workspace_bytes(N, bits))
        return fail(CGNN_EWORKSPACE, "cgnn_lsh_group: workspace too small");
    const size_t col = align_up((size_t)N * sizeof(int32_t), 256);
    char *base = static_cast<char *>(workspace);
    int32_t *rows = reinterpret_cast<int32_t *>(base);
    int32_t *sorted_code = reinterpret_cast<int32_t *>(base + col);
    int32_t *head = reinterpret_cast<int32_t *>(base + 2 * col);
    void *scan_scratch = base + 3 * col;
    void *sort_scratch = base + 3 * col + occupancy_scan_bytes(N);
    int64_t blocks = ceil_div(N, kBlock);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(iota_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, rows, N);
    size_t tb = code_sort_temp_bytes(N, bits);
    hipError_t e = hipcub::DeviceRadixSort::SortPairs(sort_scratch, tb, raw_code, sorted_code, rows, perm, (int)N,
                                                      0, bits < 1 ? 1 : bits, stream);
    if (e != hipSuccess) {
        set_error("cgnn_lsh_group: radix sort: %s", hipGetErrorString(e));
        return CGNN_ELAUNCH;
    }
    hipLaunchKernelGGL(group_heads_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, sorted_code, N, head, summary);
    int rc = occupancy_scan(head, N, sorted_id, scan_scratch, stream);
    if (rc != CGNN_OK) return rc;
    hipLaunchKernelGGL(group_finish_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, N, sorted_id, head,
                       perm, ids, offsets, summary);
    const int64_t capacity = std::min<int64_t>(N, (int64_t)1 << bits);
    int64_t cblocks = ceil_div(capacity + 1, kBlock);
    if (cblocks > 4096) cblocks = 4096;
    hipLaunchKernelGGL(group_counts_kernel, dim3((unsigned)cblocks), dim3(kBlock), 0, stream, offsets, summary,
                       counts, capacity);
    return check_launch("lsh_group");
}

extern "C" size_t cgnn_cluster_members_workspace_bytes(int64_t N, int64_t groups) {
    if (N <= 0 || groups <= 0 || N >= INT32_MAX) return 0;
    const size_t keys = align_up((size_t)N * sizeof(int32_t), 256);
    return 2 * keys + align_up(sort_temp_bytes(N, groups), 256);
}

extern "C" int cgnn_cluster_members(int64_t N, int64_t groups, const int64_t *ids, int32_t *offsets,
                                    int32_t *perm, int32_t *sorted_id, int32_t *bad_id, void *workspace,
                                    size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && groups >= 1, "cgnn_cluster_members: bad size");
    CGNN_REQUIRE(N < INT32_MAX && groups < INT32_MAX, "cgnn_cluster_members: sizes must be below 2^31");
    CGNN_REQUIRE(offsets != nullptr, "cgnn_cluster_members: offsets is null");
    int64_t oblocks = ceil_div(groups + 1, kBlock);
    if (oblocks > 4096) oblocks = 4096;
    if (N > 0) {
        CGNN_REQUIRE(ids && perm && sorted_id, "cgnn_cluster_members: null array");
        const size_t keys_bytes = align_up((size_t)N * sizeof(int32_t), 256);
        const size_t temp_bytes = sort_temp_bytes(N, groups);
        if (workspace == nullptr || workspace_bytes < 2 * keys_bytes + temp_bytes)
            return fail(CGNN_EWORKSPACE, "cgnn_cluster_members: workspace too small");
        char *base = static_cast<char *>(workspace);
        int32_t *keys = reinterpret_cast<int32_t *>(base);
        int32_t *rows = reinterpret_cast<int32_t *>(base + keys_bytes);
        void *temp = base + 2 * keys_bytes;
        int64_t blocks = ceil_div(N, kBlock);
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(members_keys_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, ids,
                           keys, rows, N, groups, bad_id);
        size_t tb = temp_bytes;
        hipError_t e = hipcub::DeviceRadixSort::SortPairs(temp, tb, keys, sorted_id, rows, perm, (int)N,
                                                          0, key_bits(groups), stream);
        if (e != hipSuccess) {
            set_error("cgnn_cluster_members: radix sort: %s", hipGetErrorString(e));
            return CGNN_ELAUNCH;
        }
    }
    hipLaunchKernelGGL(members_offsets_kernel, dim3((unsigned)oblocks), dim3(kBlock), 0, stream,
                       sorted_id, N, offsets, groups);
    return check_launch("cluster_members");
}
