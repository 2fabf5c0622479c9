// Batch pair merger on the device: the same rounds as the host routine
// cgnn_compress_csr_batch (csrc/prep.cpp), with the same arrays as result.  It stands
// where the reference's optional GPU compressor stands
// (src/offline/bindings/batch_cuda.cpp:3-9, module compressgnn_batch_cuda; its
// kernels are not part of the reference tree).
//
// A round, on the sequence of all rows laid end to end (L entries):
//   1. key[e] = (seq[e], seq[e+1]) for every e that is not the last entry of its row;
//      the keys are sorted and run-length encoded, the pairs that occur at least
//      min_pair_frequency times are the candidates, in ascending key order.
//   2. Greedy left-to-right parse of every row with all candidates.  A position is
//      "matched" if its pair is a candidate; the greedy parse takes the 1st, 3rd, 5th ...
//      position of every maximal stretch of matched positions (the last entry of a row
//      is never matched, so stretches do not cross rows).  With lz[e] = the last
//      unmatched position <= e (a running maximum), position e is taken iff it is matched
//      and e - lz[e] is odd: no sequential walk of a row, however long.
//   3. Candidates taken at least twice become rules, numbered in key order.
//   4. The parse is repeated with the rules only; taken positions emit the rule, the
//      position behind a taken one emits nothing, all others emit their entry; output
//      positions are a prefix sum, and the new row starts are the output positions of
//      the old ones.
// Sorting, run-length encoding, selection and the prefix scans are rocPRIM's (through
// hipCUB); their results do not depend on timing, the counters of step 2 are integer
// sums, so the arrays are the same run to run and equal the host routine's.
//
// Offline work: the entry point waits for the device three times per round (three
// counts decide how the round goes on).
#include <hipcub/hipcub.hpp>

#include <utility>

#include "common.h"

namespace cgnn {
namespace {

constexpr uint64_t kNoPair = ~0ull;
constexpr int64_t kMergerLimit = (int64_t)INT32_MAX - 65536;

struct MaxOp {
    __device__ __forceinline__ int32_t operator()(int32_t a, int32_t b) const { return a > b ? a : b; }
};

unsigned merger_grid(int64_t n) {
    const int64_t b = ceil_div(n, kBlock);
    return (unsigned)(b > 262144 ? 262144 : (b < 1 ? 1 : b));
}

#define CGNN_GRID_LOOP(i, n) \
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (n); i += (int64_t)gridDim.x * blockDim.x)

__global__ void merger_init_kernel(const int64_t *__restrict__ vlist, const int64_t *__restrict__ elist, int64_t V,
                                   int64_t E, int32_t *__restrict__ ptr, int32_t *__restrict__ seq,
                                   int32_t *__restrict__ bad) {
    CGNN_GRID_LOOP(i, (V + 1 > E ? V + 1 : E)) {
        if (i <= V) {
            const int64_t p = vlist[i];
            if (p < 0 || p > E || (i > 0 && p < vlist[i - 1]) || (i == 0 && p != 0) || (i == V && p != E)) *bad = 1;
            ptr[i] = (int32_t)p;
        }
        if (i < E) {
            const int64_t c = elist[i];
            if (c < 0 || c >= V) *bad = 1;
            seq[i] = (int32_t)c;
        }
    }
}

__global__ void merger_fill_kernel(int32_t *__restrict__ a, int32_t value, int64_t n) {
    CGNN_GRID_LOOP(i, n) a[i] = value;
}

// last[e] = 1 for the last entry of every non-empty row.
__global__ void merger_mark_last_kernel(const int32_t *__restrict__ ptr, int64_t V, int32_t *__restrict__ last) {
    CGNN_GRID_LOOP(v, V) {
        if (ptr[v + 1] > ptr[v]) last[ptr[v + 1] - 1] = 1;
    }
}

__global__ void merger_keys_kernel(const int32_t *__restrict__ seq, const int32_t *__restrict__ last, int64_t L,
                                   uint64_t *__restrict__ keys) {
    CGNN_GRID_LOOP(e, L) {
        keys[e] = last[e] ? kNoPair : (((uint64_t)(uint32_t)seq[e] << 32) | (uint32_t)seq[e + 1]);
    }
}

__global__ void merger_candidate_flags_kernel(const uint64_t *__restrict__ unique, const int32_t *__restrict__ counts,
                                              const int32_t *__restrict__ runs, int64_t L, int32_t min_frequency,
                                              char *__restrict__ flags) {
    const int64_t n = *runs;
    CGNN_GRID_LOOP(i, L) flags[i] = (i < n && counts[i] >= min_frequency && unique[i] != kNoPair) ? 1 : 0;
}

// idx[e] = index of key[e] among the candidates, or -1.
__global__ void merger_lookup_kernel(const uint64_t *__restrict__ keys, int64_t L,
                                     const uint64_t *__restrict__ cand, int32_t ncand, int32_t *__restrict__ idx) {
    CGNN_GRID_LOOP(e, L) {
        const uint64_t k = keys[e];
        int32_t lo = 0, hi = ncand;
        while (lo < hi) {
            const int32_t mid = (lo + hi) >> 1;
            if (cand[mid] < k) lo = mid + 1;
            else hi = mid;
        }
        idx[e] = (lo < ncand && cand[lo] == k) ? lo : -1;  // kNoPair is never a candidate
    }
}

// z[e] = e where position e is unmatched, -1 where it is matched (kept == NULL: every candidate counts).
__global__ void merger_unmatched_kernel(const int32_t *__restrict__ idx, const int32_t *__restrict__ kept,
                                        int64_t L, int32_t *__restrict__ z) {
    CGNN_GRID_LOOP(e, L) {
        const int32_t c = idx[e];
        const bool matched = c >= 0 && (kept == nullptr || kept[c] != 0);
        z[e] = matched ? -1 : (int32_t)e;
    }
}

__device__ __forceinline__ bool merger_taken(const int32_t *idx, const int32_t *kept, const int32_t *lz, int64_t e) {
    const int32_t c = idx[e];
    if (c < 0 || (kept != nullptr && kept[c] == 0)) return false;
    return ((e - (int64_t)lz[e]) & 1) != 0;
}

__global__ void merger_count_uses_kernel(const int32_t *__restrict__ idx, const int32_t *__restrict__ lz, int64_t L,
                                         int32_t *__restrict__ uses) {
    CGNN_GRID_LOOP(e, L) {
        if (merger_taken(idx, nullptr, lz, e)) atomicAdd(&uses[idx[e]], 1);
    }
}

__global__ void merger_kept_kernel(const int32_t *__restrict__ uses, int32_t ncand, int32_t *__restrict__ kept) {
    CGNN_GRID_LOOP(c, ncand) kept[c] = uses[c] >= 2 ? 1 : 0;
}

// children of the new rules, and the number of rules added (rank[c] = kept candidates before c).
__global__ void merger_rules_kernel(const uint64_t *__restrict__ cand, const int32_t *__restrict__ kept,
                                    const int32_t *__restrict__ rank, int32_t ncand, int64_t rules_before,
                                    int32_t *__restrict__ children, int32_t *__restrict__ added) {
    CGNN_GRID_LOOP(c, ncand) {
        if (kept[c]) {
            const int64_t r = rules_before + rank[c];
            children[2 * r] = (int32_t)(cand[c] >> 32);
            children[2 * r + 1] = (int32_t)(cand[c] & 0xffffffffu);
        }
        if (c == ncand - 1) *added = rank[c] + kept[c];
    }
}

__global__ void merger_emit_kernel(const int32_t *__restrict__ idx, const int32_t *__restrict__ kept,
                                   const int32_t *__restrict__ lz, int64_t L, int32_t *__restrict__ emit) {
    CGNN_GRID_LOOP(e, L) {
        const bool second = e > 0 && merger_taken(idx, kept, lz, e - 1);  // swallowed by the rule at e-1
        emit[e] = second ? 0 : 1;
    }
}

__global__ void merger_write_kernel(const int32_t *__restrict__ seq, const int32_t *__restrict__ idx,
                                    const int32_t *__restrict__ kept, const int32_t *__restrict__ rank,
                                    const int32_t *__restrict__ lz, const int32_t *__restrict__ emit,
                                    const int32_t *__restrict__ opos, int64_t L, int32_t first_new_rule,
                                    int32_t *__restrict__ out, int32_t *__restrict__ total) {
    CGNN_GRID_LOOP(e, L) {
        if (emit[e]) out[opos[e]] = merger_taken(idx, kept, lz, e) ? first_new_rule + rank[idx[e]] : seq[e];
        if (e == L - 1) *total = opos[e] + emit[e];
    }
}

__global__ void merger_new_ptr_kernel(const int32_t *__restrict__ ptr, int64_t V, int64_t L,
                                      const int32_t *__restrict__ opos, const int32_t *__restrict__ total,
                                      int32_t *__restrict__ next_ptr) {
    CGNN_GRID_LOOP(v, V + 1) next_ptr[v] = ptr[v] < L ? opos[ptr[v]] : *total;
}

// out_ptr = [row starts | starts of the rule rows], out_col = [rows | children of the rules].
__global__ void merger_finish_kernel(const int32_t *__restrict__ ptr, const int32_t *__restrict__ seq,
                                     const int32_t *__restrict__ children, int64_t V, int64_t R, int64_t L,
                                     int32_t *__restrict__ out_ptr, int32_t *__restrict__ out_col) {
    const int64_t n = L + 2 * R > V + R + 1 ? L + 2 * R : V + R + 1;
    CGNN_GRID_LOOP(i, n) {
        if (i <= V) out_ptr[i] = ptr[i];
        else if (i <= V + R) out_ptr[i] = (int32_t)(L + 2 * (i - V));
        if (i < L) out_col[i] = seq[i];
        else if (i < L + 2 * R) out_col[i] = children[i - L];
    }
}

struct MergerWorkspace {
    size_t seq[3], ptr[2], last, keys[2], counts, flags, cand, idx, z, lz, emit, opos, uses, kept, rank, children,
        scalars, temp, temp_bytes, total;
};

MergerWorkspace merger_workspace(int64_t V, int64_t E) {
    MergerWorkspace w{};
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += align_up(bytes > 0 ? bytes : 1, 256);
        return here;
    };
    const size_t n = (size_t)(E > 0 ? E : 1);
    for (auto &s : w.seq) s = take(n * 4);
    for (auto &p : w.ptr) p = take((size_t)(V + 1) * 4);
    w.last = take(n * 4);
    for (auto &k : w.keys) k = take(n * 8);  // keys[0]: keys, later the distinct keys; keys[1]: sorted keys
    w.counts = take(n * 4);
    w.flags = take(n);
    w.cand = take(n * 8);
    w.idx = take(n * 4);
    w.z = take(n * 4);
    w.lz = take(n * 4);
    w.emit = take(n * 4);
    w.opos = take(n * 4);
    w.uses = take(n * 4);
    w.kept = take(n * 4);
    w.rank = take(n * 4);
    w.children = take(n * 4);
    w.scalars = take(64);
    size_t t = 0, best = 0;
    const int m = (int)n;
    hipcub::DeviceRadixSort::SortKeys(nullptr, t, (const uint64_t *)nullptr, (uint64_t *)nullptr, m, 0, 64, 0);
    best = t > best ? t : best;
    hipcub::DeviceRunLengthEncode::Encode(nullptr, t, (const uint64_t *)nullptr, (uint64_t *)nullptr,
                                          (int32_t *)nullptr, (int32_t *)nullptr, m, 0);
    best = t > best ? t : best;
    hipcub::DeviceSelect::Flagged(nullptr, t, (const uint64_t *)nullptr, (const char *)nullptr, (uint64_t *)nullptr,
                                  (int32_t *)nullptr, m, 0);
    best = t > best ? t : best;
    hipcub::DeviceScan::InclusiveScan(nullptr, t, (const int32_t *)nullptr, (int32_t *)nullptr, MaxOp(), m, 0);
    best = t > best ? t : best;
    hipcub::DeviceScan::ExclusiveSum(nullptr, t, (const int32_t *)nullptr, (int32_t *)nullptr, m, 0);
    best = t > best ? t : best;
    w.temp_bytes = best;
    w.temp = take(best);
    w.total = at;
    return w;
}

int merger_fail(hipError_t e, const char *what) {
    set_error("cgnn_compress_csr_batch_device: %s: %s", what, hipGetErrorString(e));
    return CGNN_ELAUNCH;
}

}  // namespace
}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_compress_batch_workspace_bytes(int64_t V, int64_t E) {
    if (V < 0 || E < 0 || V >= kMergerLimit || E >= kMergerLimit) return 0;
    return merger_workspace(V, E).total;
}

extern "C" int cgnn_compress_csr_batch_device(int64_t V, int64_t E, const int64_t *vlist, const int64_t *elist,
                                              int rounds, int min_pair_frequency, int32_t *out_ptr,
                                              int32_t *out_col, int64_t *host_summary, void *workspace,
                                              size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(V >= 0 && E >= 0 && V < kMergerLimit && E < kMergerLimit,
                 "cgnn_compress_csr_batch_device: V and E must be in [0, 2^31 - 65536)");
    CGNN_REQUIRE(rounds >= 1, "cgnn_compress_csr_batch_device: rounds must be positive");
    CGNN_REQUIRE(min_pair_frequency >= 3, "cgnn_compress_csr_batch_device: min_pair_frequency must be at least 3");
    CGNN_REQUIRE(vlist && out_ptr && host_summary && (E == 0 || (elist && out_col)),
                 "cgnn_compress_csr_batch_device: null array");
    const MergerWorkspace w = merger_workspace(V, E);
    if (workspace == nullptr || workspace_bytes < w.total) {
        set_error("cgnn_compress_csr_batch_device: workspace of %zu bytes needed, %zu given", w.total, workspace_bytes);
        return CGNN_EWORKSPACE;
    }
    char *base = static_cast<char *>(workspace);
    auto i32 = [&](size_t off) { return reinterpret_cast<int32_t *>(base + off); };
    auto u64 = [&](size_t off) { return reinterpret_cast<uint64_t *>(base + off); };
    int32_t *seq = i32(w.seq[0]), *next_seq = i32(w.seq[1]);
    int32_t *ptr = i32(w.ptr[0]), *next_ptr = i32(w.ptr[1]);
    int32_t *last = i32(w.last), *counts = i32(w.counts), *idx = i32(w.idx), *z = i32(w.z), *lz = i32(w.lz);
    int32_t *emit = i32(w.emit), *opos = i32(w.opos), *uses = i32(w.uses), *kept = i32(w.kept), *rank = i32(w.rank);
    int32_t *children = i32(w.children);
    uint64_t *keys = u64(w.keys[0]), *sorted = u64(w.keys[1]), *cand = u64(w.cand);
    char *flags = base + w.flags;
    // device scalars: [0] bad input, [1] distinct keys, [2] candidates, [3] rules added, [4] new length
    int32_t *scalars = i32(w.scalars);
    void *temp = base + w.temp;
    const dim3 block(kBlock);
    auto read = [&](int k, int32_t *value) {
        hipError_t e = hipMemcpyAsync(value, scalars + k, sizeof(int32_t), hipMemcpyDeviceToHost, stream);
        if (e == hipSuccess) e = hipStreamSynchronize(stream);
        return e;
    };
    hipLaunchKernelGGL(merger_fill_kernel, dim3(1), block, 0, stream, scalars, 0, (int64_t)16);
    hipLaunchKernelGGL(merger_init_kernel, dim3(merger_grid(V + 1 > E ? V + 1 : E)), block, 0, stream, vlist, elist, V,
                       E, ptr, seq, scalars);
    int32_t bad = 0;
    hipError_t err = read(0, &bad);
    if (err != hipSuccess) return merger_fail(err, "reading the input check");
    if (bad) return fail(CGNN_EINVAL, "cgnn_compress_csr_batch_device: malformed CSR (row starts or columns out of range)");
    int64_t L = E, R = 0;
    for (int round = 0; round < rounds && L > 1; ++round) {
        const int n = (int)L;
        size_t tb = w.temp_bytes;
        hipLaunchKernelGGL(merger_fill_kernel, dim3(merger_grid(L)), block, 0, stream, last, 0, L);
        hipLaunchKernelGGL(merger_mark_last_kernel, dim3(merger_grid(V)), block, 0, stream, ptr, V, last);
        hipLaunchKernelGGL(merger_keys_kernel, dim3(merger_grid(L)), block, 0, stream, seq, last, L, keys);
        err = hipcub::DeviceRadixSort::SortKeys(temp, tb, keys, sorted, n, 0, 64, stream);
        if (err != hipSuccess) return merger_fail(err, "sort");
        uint64_t *unique = cand;  // the distinct keys; the candidates then go where the sorted keys were
        tb = w.temp_bytes;
        err = hipcub::DeviceRunLengthEncode::Encode(temp, tb, sorted, unique, counts, scalars + 1, n, stream);
        if (err != hipSuccess) return merger_fail(err, "run-length encoding");
        hipLaunchKernelGGL(merger_candidate_flags_kernel, dim3(merger_grid(L)), block, 0, stream, unique, counts,
                           scalars + 1, L, (int32_t)min_pair_frequency, flags);
        tb = w.temp_bytes;
        err = hipcub::DeviceSelect::Flagged(temp, tb, unique, flags, sorted, scalars + 2, n, stream);
        if (err != hipSuccess) return merger_fail(err, "selection");
        int32_t ncand = 0;
        if ((err = read(2, &ncand)) != hipSuccess) return merger_fail(err, "reading the candidate count");
        if (ncand == 0) break;
        const uint64_t *candidates = sorted;  // ascending
        hipLaunchKernelGGL(merger_lookup_kernel, dim3(merger_grid(L)), block, 0, stream, keys, L, candidates, ncand,
                           idx);
        // pass 1: every candidate
        hipLaunchKernelGGL(merger_unmatched_kernel, dim3(merger_grid(L)), block, 0, stream, idx,
                           (const int32_t *)nullptr, L, z);
        tb = w.temp_bytes;
        err = hipcub::DeviceScan::InclusiveScan(temp, tb, z, lz, MaxOp(), n, stream);
        if (err != hipSuccess) return merger_fail(err, "scan");
        hipLaunchKernelGGL(merger_fill_kernel, dim3(merger_grid(ncand)), block, 0, stream, uses, 0, (int64_t)ncand);
        hipLaunchKernelGGL(merger_count_uses_kernel, dim3(merger_grid(L)), block, 0, stream, idx, lz, L, uses);
        hipLaunchKernelGGL(merger_kept_kernel, dim3(merger_grid(ncand)), block, 0, stream, uses, ncand, kept);
        tb = w.temp_bytes;
        err = hipcub::DeviceScan::ExclusiveSum(temp, tb, kept, rank, ncand, stream);
        if (err != hipSuccess) return merger_fail(err, "scan");
        hipLaunchKernelGGL(merger_rules_kernel, dim3(merger_grid(ncand)), block, 0, stream, candidates, kept, rank,
                           ncand, R, children, scalars + 3);
        int32_t added = 0;
        if ((err = read(3, &added)) != hipSuccess) return merger_fail(err, "reading the rule count");
        if (added == 0) break;
        if (V + R + added >= kMergerLimit) return fail(CGNN_EUNSUPPORTED, "cgnn_compress_csr_batch_device: node ids exceed int32");
        // pass 2: the rules only
        hipLaunchKernelGGL(merger_unmatched_kernel, dim3(merger_grid(L)), block, 0, stream, idx, kept, L, z);
        tb = w.temp_bytes;
        err = hipcub::DeviceScan::InclusiveScan(temp, tb, z, lz, MaxOp(), n, stream);
        if (err != hipSuccess) return merger_fail(err, "scan");
        hipLaunchKernelGGL(merger_emit_kernel, dim3(merger_grid(L)), block, 0, stream, idx, kept, lz, L, emit);
        tb = w.temp_bytes;
        err = hipcub::DeviceScan::ExclusiveSum(temp, tb, emit, opos, n, stream);
        if (err != hipSuccess) return merger_fail(err, "scan");
        hipLaunchKernelGGL(merger_write_kernel, dim3(merger_grid(L)), block, 0, stream, seq, idx, kept, rank, lz, emit,
                           opos, L, (int32_t)(V + R), next_seq, scalars + 4);
        hipLaunchKernelGGL(merger_new_ptr_kernel, dim3(merger_grid(V + 1)), block, 0, stream, ptr, V, L, opos,
                           scalars + 4, next_ptr);
        int32_t total = 0;
        if ((err = read(4, &total)) != hipSuccess) return merger_fail(err, "reading the new length");
        std::swap(seq, next_seq);
        std::swap(ptr, next_ptr);
        L = total;
        R += added;
    }
    hipLaunchKernelGGL(merger_finish_kernel, dim3(merger_grid(L + 2 * R > V + R + 1 ? L + 2 * R : V + R + 1)), block, 0,
                       stream, ptr, seq, children, V, R, L, out_ptr, out_col);
    err = hipStreamSynchronize(stream);
    if (err != hipSuccess) return merger_fail(err, "finishing");
    host_summary[0] = R;
    host_summary[1] = L + 2 * R;
    return check_launch("compress_csr_batch_device");
}
