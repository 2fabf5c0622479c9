// The device library's own stable LSD radix sort (csrc/cluster_sort.hip), for the other files of
// the library that sort: non-negative int32 keys, the position of every key as its payload.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace cgnn {

// Bytes of counters (digit histograms per tile of keys) a sort of N keys needs.
size_t radix_sort_counter_bytes(int64_t N);

// Stable sort of (keys[i], i) by the low `bits` bits of the keys (keys >= 0): keys_out[p] is the
// p-th smallest key and pos_out[p] the index it came from; equal keys keep the order of their
// indices.  tmp_keys / tmp_pos: N entries each (used when bits > 8); counters:
// radix_sort_counter_bytes(N).  Launches on `stream`, nothing else.
int radix_sort_positions(const int32_t *keys, int64_t N, int bits, int32_t *keys_out, int32_t *pos_out,
                         int32_t *tmp_keys, int32_t *tmp_pos, void *counters, hipStream_t stream);

}  // namespace cgnn
