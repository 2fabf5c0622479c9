// Member lists of the clusters: rows sorted by cluster id, ties in ascending row
// order.  The sort itself is rocPRIM's stable LSD radix sort (through hipCUB) on
// (id, row) pairs, limited to the bits the ids occupy; it runs once per assignment
// refresh, not per training step.  Everything else here is hand-written.
#include <hipcub/hipcub.hpp>

#include "common.h"

namespace cgnn {
namespace {

__global__ void members_keys_kernel(const int64_t *__restrict__ ids, int32_t *__restrict__ keys,
                                    int32_t *__restrict__ rows, int64_t N) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
         i += (int64_t)gridDim.x * blockDim.x) {
        keys[i] = (int32_t)ids[i];
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

}  // namespace
}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_cluster_members_workspace_bytes(int64_t N, int64_t groups) {
    if (N <= 0 || groups <= 0 || N >= INT32_MAX) return 0;
    const size_t keys = align_up((size_t)N * sizeof(int32_t), 256);
    return 2 * keys + align_up(sort_temp_bytes(N, groups), 256);
}

extern "C" int cgnn_cluster_members(int64_t N, int64_t groups, const int64_t *ids, int32_t *offsets,
                                    int32_t *perm, int32_t *sorted_id, void *workspace,
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
                           keys, rows, N);
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
